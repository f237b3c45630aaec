// map_api.hip — C-ABI entry points of the map family: validation, descriptor
// lowering, dispatch. Mirrors the reference funnel (nx_c_engine.c:1362-1384):
// extract, reject packed dtypes, dispatch on the output dtype (comparisons on
// the input dtype, cast on the pair), raise statuses by kind.

#include "map_kernels.hpp"

map_launch_fn nxh_lookup_unary_a(int op, int dt);
map_launch_fn nxh_lookup_unary_b(int op, int dt);
map_launch_fn nxh_lookup_unary_c(int op, int dt);
map_launch_fn nxh_lookup_unary_d(int op, int dt);
map_launch_fn nxh_lookup_binary_a(int op, int dt);
map_launch_fn nxh_lookup_binary_b(int op, int dt);
map_launch_fn nxh_lookup_binary_c(int op, int dt);
map_launch_fn nxh_lookup_compare(int op, int dt);
map_launch_fn nxh_lookup_where(int elem_size);
map_launch_fn nxh_lookup_copy(int elem_size);
map_launch_fn nxh_lookup_cast_a(int src, int dst);
map_launch_fn nxh_lookup_cast_b(int src, int dst);
map_launch_fn nxh_lookup_cast_c(int src, int dst);
map_launch_fn nxh_lookup_cast_d(int src, int dst);

static const char *const unary_names[NXH_UNARY_COUNT] = {
    "neg",  "recip", "abs",   "sign", "sqrt",  "exp",   "log",
    "sin",  "cos",   "tan",   "asin", "acos",  "atan",  "sinh",
    "cosh", "tanh",  "trunc", "ceil", "floor", "round", "erf"};
static const char *const binary_names[NXH_BINARY_COUNT] = {
    "add", "sub", "mul", "idiv", "fdiv", "mod", "pow", "atan2", "max", "min", "xor", "or", "and"};
static const char *const compare_names[NXH_COMPARE_COUNT] = {"cmpeq", "cmpne", "cmplt", "cmple"};

// Common tail: build the plan and launch under the context lock.
static int map_run(nxh_context *ctx, const char *op, map_launch_fn fn, int dt_for_err, int nop,
                   const nxh_tensor *const *ops, const int *esize) {
  if (fn == nullptr)
    return nxh_fail(NXH_FAILURE, op, nxh_is_packed(dt_for_err) ? NXH_ERR_PACKED : NXH_ERR_UNSUPPORTED);
  for (int k = 1; k < nop; k++)
    if (!nxh_same_shape(ops[0], ops[k])) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  MapPlan p;
  int rc = map_plan_build(op, ops, nop, esize, &p);
  if (rc) return rc;
  if (p.total == 0) return NXH_OK;  // empty tensors are no-ops
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  // which operands stream past the memory-side cache: distinct bytes per operand
  const void *base[MAP_MAXOP];
  uint64_t bytes[MAP_MAXOP];
  for (int k = 0; k < nop; k++) {
    int64_t n = 1;
    for (int d = 0; d < p.ndim; d++)
      if (p.stride[k][d] != 0) n *= p.shape[d];
    base[k] = ops[k]->data;
    bytes[k] = (uint64_t)n * (uint64_t)esize[k];
  }
  p.stream = nxh_cache_hints(ctx, nop, base, bytes);
  return fn(ctx, op, p);
}

#define NXH_CHECK_ARGS(op, ...)                                                    \
  do {                                                                             \
    if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null context");           \
    const nxh_tensor *ts__[] = {__VA_ARGS__};                                      \
    for (const nxh_tensor *t__ : ts__) {                                           \
      if (!t__) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null tensor");          \
      int rc__ = nxh_check_tensor(op, t__);                                        \
      if (rc__) return rc__;                                                       \
    }                                                                              \
  } while (0)

NXH_EXPORT int nxh_unary(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x) {
  if ((unsigned)op >= NXH_UNARY_COUNT) return nxh_fail(NXH_INVALID_ARGUMENT, "unary", "unknown op");
  const char *name = unary_names[op];
  NXH_CHECK_ARGS(name, out, x);
  NXH_DEFER_RECORD(ctx, NXH_D_UNARY, op, out, 1, nullptr, 0, nullptr, x);
  const int dt = out->dtype;
  if (nxh_is_packed(dt) || nxh_is_packed(x->dtype)) return nxh_fail(NXH_FAILURE, name, NXH_ERR_PACKED);
  if (x->dtype != dt) return nxh_fail(NXH_FAILURE, name, NXH_ERR_UNSUPPORTED);
  map_launch_fn fn = nxh_lookup_unary_a(op, dt);
  if (!fn) fn = nxh_lookup_unary_b(op, dt);
  if (!fn) fn = nxh_lookup_unary_c(op, dt);
  if (!fn) fn = nxh_lookup_unary_d(op, dt);
  const nxh_tensor *ops[2] = {out, x};
  const int es[2] = {(int)nxh_elem_size(dt), (int)nxh_elem_size(dt)};
  return map_run(ctx, name, fn, dt, 2, ops, es);
}

NXH_EXPORT int nxh_binary(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x,
                          const nxh_tensor *y) {
  if ((unsigned)op >= NXH_BINARY_COUNT) return nxh_fail(NXH_INVALID_ARGUMENT, "binary", "unknown op");
  const char *name = binary_names[op];
  NXH_CHECK_ARGS(name, out, x, y);
  NXH_DEFER_RECORD(ctx, NXH_D_BINARY, op, out, 2, nullptr, 0, nullptr, x, y);
  const int dt = out->dtype;
  if (nxh_is_packed(dt) || nxh_is_packed(x->dtype) || nxh_is_packed(y->dtype))
    return nxh_fail(NXH_FAILURE, name, NXH_ERR_PACKED);
  if (x->dtype != dt || y->dtype != dt) return nxh_fail(NXH_FAILURE, name, NXH_ERR_UNSUPPORTED);
  map_launch_fn fn = nxh_lookup_binary_a(op, dt);
  if (!fn) fn = nxh_lookup_binary_b(op, dt);
  if (!fn) fn = nxh_lookup_binary_c(op, dt);
  const nxh_tensor *ops[3] = {out, x, y};
  const int e = (int)nxh_elem_size(dt);
  const int es[3] = {e, e, e};
  return map_run(ctx, name, fn, dt, 3, ops, es);
}

NXH_EXPORT int nxh_compare(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x,
                           const nxh_tensor *y) {
  if ((unsigned)op >= NXH_COMPARE_COUNT) return nxh_fail(NXH_INVALID_ARGUMENT, "compare", "unknown op");
  const char *name = compare_names[op];
  NXH_CHECK_ARGS(name, out, x, y);
  NXH_DEFER_RECORD(ctx, NXH_D_COMPARE, op, out, 2, nullptr, 0, nullptr, x, y);
  const int dt = x->dtype;
  if (nxh_is_packed(dt) || nxh_is_packed(y->dtype)) return nxh_fail(NXH_FAILURE, name, NXH_ERR_PACKED);
  if (y->dtype != dt || nxh_elem_size(out->dtype) != 1)
    return nxh_fail(NXH_FAILURE, name, NXH_ERR_UNSUPPORTED);
  map_launch_fn fn = nxh_lookup_compare(op, dt);
  const nxh_tensor *ops[3] = {out, x, y};
  const int e = (int)nxh_elem_size(dt);
  const int es[3] = {1, e, e};
  return map_run(ctx, name, fn, dt, 3, ops, es);
}

NXH_EXPORT int nxh_where(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *cond,
                         const nxh_tensor *a, const nxh_tensor *b) {
  NXH_CHECK_ARGS("where", out, cond, a, b);
  NXH_DEFER_RECORD(ctx, NXH_D_WHERE, 0, out, 3, nullptr, 0, nullptr, cond, a, b);
  const int dt = out->dtype;
  if (nxh_is_packed(dt)) return nxh_fail(NXH_FAILURE, "where", NXH_ERR_PACKED);
  if (a->dtype != dt || b->dtype != dt || nxh_elem_size(cond->dtype) != 1)
    return nxh_fail(NXH_FAILURE, "where", NXH_ERR_UNSUPPORTED);
  const int e = (int)nxh_elem_size(dt);
  const nxh_tensor *ops[4] = {out, cond, a, b};
  const int es[4] = {e, 1, e, e};
  return map_run(ctx, "where", nxh_lookup_where(e), dt, 4, ops, es);
}

struct alignas(16) B16x {
  uint64_t lo, hi;
};
static int copy_impl(nxh_context *ctx, const char *op, const nxh_tensor *out, const nxh_tensor *x);

NXH_EXPORT int nxh_copy(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x) {
  if (out && x && !nxh_is_packed(out->dtype) && !nxh_is_packed(x->dtype)) {
    NXH_DEFER_RECORD(ctx, NXH_D_COPY, 0, out, 1, nullptr, 0, nullptr, x);
  } else {
    NXH_DEFER_TOUCH(ctx, 1, out, x);
  }
  NXH_CHECK_ARGS("copy", out, x);
  return copy_impl(ctx, "copy", out, x);
}

// ── packed int4 / uint4 (nx_c_map.c:1046-1177; nx_c_move.c:143-189) ─────────
// Storage-only dtypes: dense layouts, cast and whole-buffer copy only. Element i
// of a packed operand is nibble (offset + i), low nibble first.
__device__ static bool packed_read(int dt, const void *base, int64_t e, int64_t *iv, double *fv) {
  switch (dt) {
    case NXH_F16: *fv = (double)f16_to_f32(((const uint16_t *)base)[e]); return true;
    case NXH_BF16: *fv = (double)bf16_to_f32(((const uint16_t *)base)[e]); return true;
    case NXH_F32: *fv = (double)((const float *)base)[e]; return true;
    case NXH_F64: *fv = ((const double *)base)[e]; return true;
    case NXH_F8E4M3: *fv = (double)f8e4m3_to_f32(((const uint8_t *)base)[e]); return true;
    case NXH_F8E5M2: *fv = (double)f8e5m2_to_f32(((const uint8_t *)base)[e]); return true;
    case NXH_C32: *fv = (double)((const c32 *)base)[e].re; return true;
    case NXH_C64: *fv = ((const c64 *)base)[e].re; return true;
    case NXH_I8: *iv = ((const int8_t *)base)[e]; return false;
    case NXH_U8: *iv = ((const uint8_t *)base)[e]; return false;
    case NXH_I16: *iv = ((const int16_t *)base)[e]; return false;
    case NXH_U16: *iv = ((const uint16_t *)base)[e]; return false;
    case NXH_I32: *iv = ((const int32_t *)base)[e]; return false;
    case NXH_U32: *iv = ((const uint32_t *)base)[e]; return false;
    case NXH_I64: *iv = ((const int64_t *)base)[e]; return false;
    case NXH_U64: *iv = (int64_t)((const uint64_t *)base)[e]; return false;
    case NXH_BOOL: *iv = ((const uint8_t *)base)[e] != 0; return false;
    default: *iv = 0; return false;
  }
}
__device__ static uint8_t nibble_of(int dst, int src, const void *sbase, int64_t soff, int64_t i) {
  if (src == NXH_I4 || src == NXH_U4) {
    int64_t si = soff + i;
    uint8_t by = ((const uint8_t *)sbase)[si >> 1];
    return (uint8_t)((by >> ((si & 1) * 4)) & 0x0f);
  }
  int64_t iv = 0;
  double fv = 0;
  bool isf = packed_read(src, sbase, soff + i, &iv, &fv);
  int v;
  if (isf) {
    if (fv != fv) v = 0;
    else if (dst == NXH_I4) v = fv <= -8.0 ? -8 : (fv >= 7.0 ? 7 : (int)fv);
    else v = fv <= 0.0 ? 0 : (fv >= 15.0 ? 15 : (int)fv);
  } else {
    v = (int)iv;
  }
  return (uint8_t)v & 0x0f;
}
// One thread per destination BYTE, so the two nibbles of a byte never race.
__global__ void cast_to_packed_kernel(uint8_t *dbase, int64_t doff, int dst, const void *sbase,
                                      int64_t soff, int src, int64_t n) {
  int64_t first_byte = doff >> 1, last_byte = (doff + n - 1) >> 1;
  int64_t b = first_byte + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > last_byte) return;
  uint8_t cur = dbase[b];
  for (int h = 0; h < 2; h++) {
    int64_t di = b * 2 + h, i = di - doff;
    if (i < 0 || i >= n) continue;
    uint8_t nib = nibble_of(dst, src, sbase, soff, i);
    cur = h ? (uint8_t)((cur & 0x0f) | (nib << 4)) : (uint8_t)((cur & 0xf0) | nib);
  }
  dbase[b] = cur;
}
template <int DST>
__device__ static void packed_store(void *dbase, int64_t e, int64_t v) {
  using T = Tr<DST>;
  using DC = typename T::C;
  typename T::S *p = (typename T::S *)dbase + e;
  if constexpr (T::cat == CAT_COMPLEX) {
    using R = decltype(DC{}.re);
    *p = T::st(DC{(R)v, (R)0});
  } else if constexpr (T::cat == CAT_BOOL) *p = T::st((DC)(v != 0));
  else *p = T::st((DC)v);
}
__global__ void cast_from_packed_kernel(void *dbase, int64_t doff, int dst, const uint8_t *sbase,
                                        int64_t soff, int src, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int64_t si = soff + i;
  uint8_t by = sbase[si >> 1];
  int64_t v = src == NXH_I4 ? ((si & 1) ? ((int8_t)by >> 4) : ((int8_t)((by & 0x0f) << 4) >> 4))
                            : ((si & 1) ? (by >> 4) : (by & 0x0f));
  switch (dst) {
#define NXH_CASE(DT) \
  case DT: packed_store<DT>(dbase, doff + i, v); break;
    NXH_FOR_COMPUTE_DTYPES(NXH_CASE)
#undef NXH_CASE
    default: break;
  }
}

static bool dense_layout(const nxh_tensor *a) {
  int64_t e = 1;
  for (int i = a->ndim - 1; i >= 0; i--) {
    if (a->shape[i] == 1) continue;
    if (a->strides[i] != e) return false;
    e *= a->shape[i];
  }
  return true;
}

static int cast_packed(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x) {
  if (!dense_layout(out) || !dense_layout(x)) return nxh_fail(NXH_FAILURE, "cast", NXH_ERR_PACKED);
  int64_t n = 1;
  for (int i = 0; i < out->ndim; i++) n *= out->shape[i];
  if (n == 0) return NXH_OK;
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("cast", hipSetDevice(ctx->device));
  nxh_set_path("cast_packed");
  if (nxh_is_packed(out->dtype)) {
    int64_t bytes = ((out->offset + n - 1) >> 1) - (out->offset >> 1) + 1;
    hipLaunchKernelGGL(cast_to_packed_kernel, dim3((unsigned)((bytes + 255) / 256)), dim3(256), 0,
                       ctx->stream, (uint8_t *)out->data, out->offset, out->dtype, x->data,
                       x->offset, x->dtype, n);
  } else {
    hipLaunchKernelGGL(cast_from_packed_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       ctx->stream, out->data, out->offset, out->dtype, (const uint8_t *)x->data,
                       x->offset, x->dtype, n);
  }
  NXH_HIP("cast", hipGetLastError());
  return NXH_OK;
}

NXH_EXPORT int nxh_cast(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x) {
  NXH_CHECK_ARGS("cast", out, x);
  if (!nxh_same_shape(out, x)) return nxh_fail(NXH_INVALID_ARGUMENT, "cast", NXH_ERR_SHAPE);
  const int src = x->dtype, dst = out->dtype;
  if (nxh_is_packed(src) || nxh_is_packed(dst)) {
    NXH_DEFER_TOUCH(ctx, 1, out, x);
    return cast_packed(ctx, out, x);
  }
  NXH_DEFER_RECORD(ctx, NXH_D_CAST, 0, out, 1, nullptr, 0, nullptr, x);
  map_launch_fn fn = nxh_lookup_cast_a(src, dst);
  if (!fn) fn = nxh_lookup_cast_b(src, dst);
  if (!fn) fn = nxh_lookup_cast_c(src, dst);
  if (!fn) fn = nxh_lookup_cast_d(src, dst);
  const nxh_tensor *ops[2] = {out, x};
  const int es[2] = {(int)nxh_elem_size(dst), (int)nxh_elem_size(src)};
  return map_run(ctx, "cast", fn, dst, 2, ops, es);
}

// copy / contiguous / assign (nx_c_move.c:191-201). Packed dtypes: whole
// contiguous offset-0 buffers only, copied as bytes with the odd trailing
// nibble merged (nx_c_move.c:143-189).
__global__ void merge_low_nibble_kernel(uint8_t *d, const uint8_t *s) {
  *d = (uint8_t)((*d & 0xf0) | (*s & 0x0f));
}
static int copy_impl(nxh_context *ctx, const char *op, const nxh_tensor *out, const nxh_tensor *x) {
  const int dt = out->dtype;
  if (x->dtype != dt) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (nxh_is_packed(dt)) {
    int64_t n = 1, nx = 1;
    for (int i = 0; i < out->ndim; i++) n *= out->shape[i];
    for (int i = 0; i < x->ndim; i++) nx *= x->shape[i];
    if (n != nx || !dense_layout(out) || !dense_layout(x) || out->offset != 0 || x->offset != 0)
      return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
    std::lock_guard<std::mutex> g(ctx->mu);
    NXH_HIP(op, hipSetDevice(ctx->device));
    if (n / 2 > 0)
      NXH_HIP(op, hipMemcpyAsync(out->data, x->data, (size_t)(n / 2), hipMemcpyDeviceToDevice, ctx->stream));
    if (n & 1) {
      hipLaunchKernelGGL(merge_low_nibble_kernel, dim3(1), dim3(1), 0, ctx->stream,
                         (uint8_t *)out->data + n / 2, (const uint8_t *)x->data + n / 2);
      NXH_HIP(op, hipGetLastError());
    }
    return NXH_OK;
  }
  const int e = (int)nxh_elem_size(dt);
  const nxh_tensor *ops[2] = {out, x};
  const int es[2] = {e, e};
  return map_run(ctx, op, nxh_lookup_copy(e), dt, 2, ops, es);
}

// full (nx_backend.ml:61-64). The encoded element travels as a kernel argument,
// so the call needs no host->device copy and no wait. A contiguous destination
// (every `full` result) takes the 16-byte-store kernel; any other layout seeds a
// one-element device block and broadcasts it through the copy kernel with a
// stride-0 source, the way the reference passes pad's fill value as a
// one-element tensor (nx_backend.ml:362-373).
struct FillValue {
  uint64_t w[2];
};
__global__ void seed_value_kernel(uint64_t *dst, FillValue v) {
  dst[0] = v.w[0];
  dst[1] = v.w[1];
}
// `pattern` holds the element replicated across 16 bytes.
__global__ __launch_bounds__(256) void fill_contig_kernel(uint8_t *out, int64_t bytes, FillValue pattern) {
  const int64_t nvec = bytes / 16;
  B16x *o = reinterpret_cast<B16x *>(out);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec;
       i += (int64_t)gridDim.x * blockDim.x)
    o[i] = B16x{pattern.w[0], pattern.w[1]};
  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(bytes - nvec * 16)) {
    const uint8_t *pb = reinterpret_cast<const uint8_t *>(&pattern);
    out[nvec * 16 + threadIdx.x] = pb[threadIdx.x];
  }
}

NXH_EXPORT int nxh_fill(nxh_context *ctx, const nxh_tensor *out, const void *value) {
  NXH_CHECK_ARGS("full", out);
  if (!value) return nxh_fail(NXH_INVALID_ARGUMENT, "full", "null value");
  if (nxh_defer_active(ctx)) {
    // a one-element fill is recorded (the scalars of a fused run are then never filled on the
    // device); any other fill runs the record first
    const int drc = nxh_defer_record(ctx, NXH_D_FULL, 0, out, nullptr, 0, nullptr, 0, value);
    if (drc != -1) return drc;
  }
  const int dt = out->dtype;
  int64_t n = 1;
  for (int i = 0; i < out->ndim; i++) n *= out->shape[i];
  if (nxh_is_packed(dt)) {
    // both nibbles of every byte take the low nibble of *value
    if (!dense_layout(out) || out->offset != 0) return nxh_fail(NXH_FAILURE, "full", NXH_ERR_PACKED);
    uint8_t nib = *(const uint8_t *)value & 0x0f;
    FillValue pat;
    memset(&pat, nib | (nib << 4), sizeof pat);
    if (n == 0) return NXH_OK;
    std::lock_guard<std::mutex> g(ctx->mu);
    NXH_HIP("full", hipSetDevice(ctx->device));
    hipLaunchKernelGGL(fill_contig_kernel, dim3(1), dim3(256), 0, ctx->stream, (uint8_t *)out->data,
                       (n + 1) / 2, pat);
    NXH_HIP("full", hipGetLastError());
    return NXH_OK;
  }
  if (n == 0) return NXH_OK;
  const int e = (int)nxh_elem_size(dt);
  FillValue pat;
  for (int i = 0; i < 16; i += e) memcpy((char *)&pat + i, value, (size_t)e);
  char *first = (char *)out->data + out->offset * e;
  if (dense_layout(out) && aligned_to(first, 16)) {
    const int64_t bytes = n * e;
    int64_t blocks = (bytes / 16 + 255) / 256;
    blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, 256 * 32));
    std::lock_guard<std::mutex> g(ctx->mu);
    NXH_HIP("full", hipSetDevice(ctx->device));
    nxh_set_path("fill_contig");
    hipLaunchKernelGGL(fill_contig_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       (uint8_t *)first, bytes, pat);
    NXH_HIP("full", hipGetLastError());
    return NXH_OK;
  }
  void *staged = nullptr;
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    NXH_HIP("full", hipSetDevice(ctx->device));
    int rc = nxh_alloc_locked(ctx, 16, &staged);
    if (rc) return rc;
    hipLaunchKernelGGL(seed_value_kernel, dim3(1), dim3(1), 0, ctx->stream, (uint64_t *)staged, pat);
  }
  nxh_tensor src = *out;
  src.data = staged;
  src.offset = 0;
  for (int i = 0; i < src.ndim; i++) src.strides[i] = 0;
  int rc = copy_impl(ctx, "full", out, &src);
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    nxh_free_locked(ctx, staged);  // stream-ordered: the copy kernel is already queued
  }
  return rc;
}
