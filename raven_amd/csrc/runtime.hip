// runtime.hip — context, caching device allocator, host<->device transfer,
// status protocol and timing for libnxhip.
//
// What it replaces in the reference: Nx_buffer allocation inside
// nx_backend.ml:54-69 (buffer / full / from_host / to_host), the status ->
// exception funnel of nx_c_engine.c:42-52,1345-1351, and create_context
// (nx_backend.mli:32-39). There is no thread pool: one HIP stream per context
// orders all work, and blocks returned to the allocator are reused only by
// later work on that same stream.

#include <cstdlib>

#include "nxh_common.hpp"

static thread_local char tls_error[512] = "";
static thread_local const char *tls_path = "";

void nxh_set_error(const char *op, const char *msg) {
  snprintf(tls_error, sizeof tls_error, "%s: %s", op, msg);
}
void nxh_set_path(const char *path) { tls_path = path; }
int nxh_fail(int kind, const char *op, const char *msg) {
  nxh_set_error(op, msg);
  return kind;
}
int nxh_hip_fail(const char *op, hipError_t e) {
  // Device-runtime errors are Failure, like the reference's non-argument
  // statuses (nx_c_engine.c:1345-1351).
  char buf[256];
  snprintf(buf, sizeof buf, "HIP error %d (%s)", (int)e, hipGetErrorString(e));
  (void)hipGetLastError();  // clear the sticky error so later calls report their own
  return nxh_fail(NXH_FAILURE, op, buf);
}

NXH_EXPORT const char *nxh_last_error(nxh_context *) { return tls_error; }
NXH_EXPORT const char *nxh_last_path(nxh_context *) { return tls_path; }

NXH_EXPORT int nxh_context_create(nxh_context **out) {
  if (!out) return nxh_fail(NXH_INVALID_ARGUMENT, "create_context", "null output pointer");
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0) {
    (void)hipGetLastError();
    return nxh_fail(NXH_FAILURE, "create_context", "no HIP device available");
  }
  int dev = 0;
  if (const char *s = getenv("NX_HIP_DEVICE")) dev = atoi(s);
  if (dev < 0 || dev >= count)
    return nxh_fail(NXH_FAILURE, "create_context", "NX_HIP_DEVICE out of range");
  NXH_HIP("create_context", hipSetDevice(dev));
  nxh_context *ctx = new nxh_context();
  ctx->device = dev;
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e == hipSuccess) {
    ctx->compute_units = prop.multiProcessorCount;
    snprintf(ctx->name, sizeof ctx->name, "%s (%s)", prop.name, prop.gcnArchName);
  }
  // default priority, non-blocking with respect to the legacy stream
  e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipEventCreate(&ctx->ev_start);
  if (e == hipSuccess) e = hipEventCreate(&ctx->ev_stop);
  if (e == hipSuccess) e = hipMalloc((void **)&ctx->fault_flag, 256);
  if (e == hipSuccess) e = hipHostMalloc((void **)&ctx->fault_flag_host, 256, hipHostMallocDefault);
  if (e == hipSuccess)
    e = hipHostMalloc((void **)&ctx->stage, nxh_context::STAGE_SLOTS * nxh_context::STAGE_BYTES, hipHostMallocDefault);
  for (int i = 0; i < nxh_context::STAGE_SLOTS && e == hipSuccess; i++)
    e = hipEventCreateWithFlags(&ctx->stage_done[i], hipEventDisableTiming);
  if (e == hipSuccess) e = hipMemsetAsync(ctx->fault_flag, 0, 256, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) {
    delete ctx;
    return nxh_hip_fail("create_context", e);
  }
  *out = ctx;
  return NXH_OK;
}

NXH_EXPORT void nxh_context_destroy(nxh_context *ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  for (auto &kv : ctx->live) (void)hipFree(kv.first);
  if (ctx->fault_flag) (void)hipFree(ctx->fault_flag);
  if (ctx->fault_flag_host) (void)hipHostFree(ctx->fault_flag_host);
  if (ctx->stage) (void)hipHostFree(ctx->stage);
  for (hipEvent_t ev : ctx->stage_done)
    if (ev) (void)hipEventDestroy(ev);
  if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
  if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

NXH_EXPORT int nxh_device_info(nxh_context *ctx, int *device, char *name, size_t name_len,
                               int *compute_units) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "device_info", "null context");
  if (device) *device = ctx->device;
  if (name && name_len) snprintf(name, name_len, "%s", ctx->name);
  if (compute_units) *compute_units = ctx->compute_units;
  return NXH_OK;
}

NXH_EXPORT int64_t nxh_dtype_bytes(int dtype, int64_t count) {
  if ((unsigned)dtype >= NXH_DTYPE_COUNT || count < 0) return -1;
  if (nxh_is_packed(dtype)) return (count + 1) / 2;
  return count * nxh_elem_size(dtype);
}

// ── caching allocator ──────────────────────────────────────────────────────
// Size classes: 512 B granules up to 1 MiB, then 1/8-octave steps (<= 12.5 %
// slack). The eager frontend allocates one output per primitive (about a
// thousand per GPT-2 forward), so hipMalloc/hipFree never sit on that path once
// the working set has been seen. Every block is 256-byte aligned, exact-size
// from the caller's point of view, and never a sub-range of another block.
static size_t size_class(size_t bytes) {
  if (bytes == 0) bytes = 1;
  if (bytes <= ((size_t)1 << 20)) return (bytes + 511) & ~(size_t)511;
  int top = 63 - __builtin_clzll((unsigned long long)bytes);
  size_t step = (size_t)1 << (top - 3);
  return (bytes + step - 1) & ~(step - 1);
}

int nxh_alloc_locked(nxh_context *ctx, size_t bytes, void **out) {
  size_t cls = size_class(bytes);
  auto it = ctx->free_lists.find(cls);
  if (it != ctx->free_lists.end() && !it->second.empty()) {
    *out = it->second.back();
    it->second.pop_back();
    ctx->cached -= cls;
    ctx->in_use += cls;
    return NXH_OK;
  }
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, cls);
  if (e != hipSuccess) {
    // give cached blocks back to the driver and retry once
    (void)hipGetLastError();
    (void)hipStreamSynchronize(ctx->stream);
    for (auto &kv : ctx->free_lists) {
      for (void *q : kv.second) {
        (void)hipFree(q);
        ctx->live.erase(q);
        ctx->reserved -= kv.first;
        ctx->cached -= kv.first;
      }
      kv.second.clear();
    }
    e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return nxh_fail(NXH_FAILURE, "buffer", NXH_ERR_ALLOC);
    }
  }
  ctx->live[p] = cls;
  ctx->reserved += cls;
  ctx->in_use += cls;
  ctx->driver_allocs++;
  *out = p;
  return NXH_OK;
}

void nxh_free_locked(nxh_context *ctx, void *p) {
  auto it = ctx->live.find(p);
  if (it == ctx->live.end()) return;
  ctx->free_lists[it->second].push_back(p);
  ctx->in_use -= it->second;
  ctx->cached += it->second;
}

NXH_EXPORT int nxh_alloc(nxh_context *ctx, size_t bytes, void **dptr) {
  if (!ctx || !dptr) return nxh_fail(NXH_INVALID_ARGUMENT, "buffer", "null argument");
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("buffer", hipSetDevice(ctx->device));
  return nxh_alloc_locked(ctx, bytes, dptr);
}

NXH_EXPORT int nxh_free(nxh_context *ctx, void *dptr) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "free", "null context");
  if (!dptr) return NXH_OK;
  std::lock_guard<std::mutex> g(ctx->mu);
  if (ctx->live.find(dptr) == ctx->live.end())
    return nxh_fail(NXH_INVALID_ARGUMENT, "free", "pointer not owned by this context");
  nxh_free_locked(ctx, dptr);
  return NXH_OK;
}

NXH_EXPORT int nxh_trim(nxh_context *ctx) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "trim", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("trim", hipSetDevice(ctx->device));
  NXH_HIP("trim", hipStreamSynchronize(ctx->stream));
  for (auto &kv : ctx->free_lists) {
    for (void *q : kv.second) {
      (void)hipFree(q);
      ctx->live.erase(q);
      ctx->reserved -= kv.first;
      ctx->cached -= kv.first;
    }
    kv.second.clear();
  }
  return NXH_OK;
}

NXH_EXPORT int nxh_memory_stats(nxh_context *ctx, uint64_t *in_use, uint64_t *cached,
                                uint64_t *reserved, uint64_t *driver_allocs) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "memory_stats", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (in_use) *in_use = ctx->in_use;
  if (cached) *cached = ctx->cached;
  if (reserved) *reserved = ctx->reserved;
  if (driver_allocs) *driver_allocs = ctx->driver_allocs;
  return NXH_OK;
}

// ── transfer ───────────────────────────────────────────────────────────────
// from_host must not return before the caller's buffer has been read: the
// frontend fills a temporary and drops it (frontend.ml:347-351). Uploads of up
// to 256 KiB (index vectors, aranges, scalars) are copied into a pinned slot
// of the context and queued, so they do not drain the stream; larger ones are
// queued from the caller's buffer and waited for.
NXH_EXPORT int nxh_memcpy_h2d(nxh_context *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "from_host", "null context");
  if (bytes == 0) return NXH_OK;
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("from_host", hipSetDevice(ctx->device));
  if (bytes <= nxh_context::STAGE_BYTES) {
    // small upload: through a pinned slot, in stream order, without waiting
    // for the stream. A slot is reused only after its last transfer finished.
    const int slot = ctx->stage_next;
    ctx->stage_next = (slot + 1) % nxh_context::STAGE_SLOTS;
    if (ctx->stage_used[slot]) NXH_HIP("from_host", hipEventSynchronize(ctx->stage_done[slot]));
    char *staged = ctx->stage + (size_t)slot * nxh_context::STAGE_BYTES;
    memcpy(staged, src, bytes);
    NXH_HIP("from_host", hipMemcpyAsync(dst, staged, bytes, hipMemcpyHostToDevice, ctx->stream));
    NXH_HIP("from_host", hipEventRecord(ctx->stage_done[slot], ctx->stream));
    ctx->stage_used[slot] = true;
    return NXH_OK;
  }
  NXH_HIP("from_host", hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  NXH_HIP("from_host", hipStreamSynchronize(ctx->stream));
  return NXH_OK;
}

NXH_EXPORT int nxh_memcpy_d2h(nxh_context *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "to_host", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("to_host", hipSetDevice(ctx->device));
  if (bytes)
    NXH_HIP("to_host", hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  NXH_HIP("to_host", hipStreamSynchronize(ctx->stream));
  return NXH_OK;
}

NXH_EXPORT int nxh_synchronize(nxh_context *ctx) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "synchronize", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("synchronize", hipSetDevice(ctx->device));
  NXH_HIP("synchronize", hipStreamSynchronize(ctx->stream));
  return NXH_OK;
}

// ── timing ─────────────────────────────────────────────────────────────────
NXH_EXPORT int nxh_timer_start(nxh_context *ctx) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "timer", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("timer", hipEventRecord(ctx->ev_start, ctx->stream));
  return NXH_OK;
}
NXH_EXPORT int nxh_timer_stop(nxh_context *ctx, float *ms) {
  if (!ctx || !ms) return nxh_fail(NXH_INVALID_ARGUMENT, "timer", "null argument");
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP("timer", hipEventRecord(ctx->ev_stop, ctx->stream));
  NXH_HIP("timer", hipEventSynchronize(ctx->ev_stop));
  NXH_HIP("timer", hipEventElapsedTime(ms, ctx->ev_start, ctx->ev_stop));
  return NXH_OK;
}
