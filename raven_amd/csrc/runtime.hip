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

// ── static workspace ───────────────────────────────────────────────────────
// Device memory that exists from the moment the code object is loaded, one copy
// per GPU, for the entry point that must not allocate (nxh_reduce_noalloc keeps
// the partial results of a split reduction here). In host code the array's name
// is only a handle for hipGetSymbolAddress: the device address is looked up once
// per device, with that device current, and every launch is given that address.
static __device__ __align__(256) unsigned char scratch[NXH_STATIC_WS_BYTES];

static std::mutex scratch_mu;
static unsigned char *scratch_ptr[64] = {};

static hipError_t static_workspace(int device, unsigned char **out) {
  std::lock_guard<std::mutex> g(scratch_mu);
  if ((unsigned)device >= 64) return hipErrorInvalidDevice;
  if (!scratch_ptr[device]) {
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    scratch_ptr[device] = (unsigned char *)p;
  }
  *out = scratch_ptr[device];
  return hipSuccess;
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
  if (e == hipSuccess) e = static_workspace(dev, &ctx->static_ws);  // device `dev` is current
  if (const char *s = getenv("NXH_CACHE_HINTS")) ctx->cache_hints = atoi(s) & 7;
  if (e != hipSuccess) {
    delete ctx;
    return nxh_hip_fail("create_context", e);
  }
  *out = ctx;
  return NXH_OK;
}

NXH_EXPORT void nxh_context_destroy(nxh_context *ctx) {
  if (!ctx) return;
  nxh_defer_context_gone(ctx);
  (void)hipSetDevice(ctx->device);
  if (ctx->capture) {  // abandoned capture: close it so the stream can be destroyed
    hipGraph_t dropped = nullptr;
    (void)hipStreamEndCapture(ctx->stream, &dropped);
    if (dropped) (void)hipGraphDestroy(dropped);
    (void)hipGetLastError();
  }
  (void)hipStreamSynchronize(ctx->stream);
  for (auto &kv : ctx->live) (void)hipFree(kv.first);
  for (auto &kv : ctx->device_tables) (void)hipFree(kv.second);
  if (ctx->fault_flag) (void)hipFree(ctx->fault_flag);
  if (ctx->scan_state) (void)hipFree(ctx->scan_state);
  for (void *t : ctx->gelu_lut)
    if (t) (void)hipFree(t);
  if (ctx->gelu_epi.dev) (void)hipFree(ctx->gelu_epi.dev);
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
static int refuse_while_capturing(nxh_context *ctx, const char *op) {
  if (ctx->capture) return nxh_fail(NXH_FAILURE, op, "not allowed while a graph is being captured");
  return NXH_OK;
}

static size_t size_class(size_t bytes) {
  if (bytes == 0) bytes = 1;
  if (bytes <= ((size_t)1 << 20)) return (bytes + 511) & ~(size_t)511;
  int top = 63 - __builtin_clzll((unsigned long long)bytes);
  size_t step = (size_t)1 << (top - 3);
  return (bytes + step - 1) & ~(step - 1);
}

int nxh_alloc_locked(nxh_context *ctx, size_t bytes, void **out) {
  size_t cls = size_class(bytes);
  nxh_graph *cap = ctx->capture;
  if (cap) {  // a block the graph already holds, before anything else
    auto git = cap->free_lists.find(cls);
    if (git != cap->free_lists.end() && !git->second.empty()) {
      *out = git->second.back();
      git->second.pop_back();
      ctx->in_use += cls;
      return NXH_OK;
    }
  }
  auto it = ctx->free_lists.find(cls);
  if (it != ctx->free_lists.end() && !it->second.empty()) {
    *out = it->second.back();
    it->second.pop_back();
    ctx->cached -= cls;
    ctx->in_use += cls;
    if (cap) ctx->graph_blocks[*out] = cap;  // from now on the graph's
    return NXH_OK;
  }
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, cls);
  if (e != hipSuccess && !cap) {
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
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return nxh_fail(NXH_FAILURE, "buffer", NXH_ERR_ALLOC);
  }
  ctx->live[p] = cls;
  ctx->reserved += cls;
  ctx->in_use += cls;
  ctx->driver_allocs++;
  if (cap) ctx->graph_blocks[p] = cap;
  *out = p;
  return NXH_OK;
}

void nxh_free_locked(nxh_context *ctx, void *p) {
  auto it = ctx->live.find(p);
  if (it == ctx->live.end()) return;
  ctx->in_use -= it->second;
  // a block a graph holds stays with that graph (its replays write there): it is
  // reused only by later allocations of the same capture
  auto g = ctx->graph_blocks.find(p);
  if (g != ctx->graph_blocks.end()) {
    g->second->free_lists[it->second].push_back(p);
    return;
  }
  ctx->free_lists[it->second].push_back(p);
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
  if (nxh_defer_free(ctx, dptr)) return NXH_OK;  // recorded entries still use the block: freed once they have run
  std::lock_guard<std::mutex> g(ctx->mu);
  if (ctx->live.find(dptr) == ctx->live.end())
    return nxh_fail(NXH_INVALID_ARGUMENT, "free", "pointer not owned by this context");
  nxh_free_locked(ctx, dptr);
  return NXH_OK;
}

NXH_EXPORT int nxh_trim(nxh_context *ctx) {
  NXH_DEFER_QUIET(ctx);
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "trim", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (int rc = refuse_while_capturing(ctx, "trim")) return rc;
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
  ctx->block_use.clear();  // addresses may come back as other blocks
  for (const void *&b : ctx->recent_block) b = nullptr;
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

// ── cache hints ────────────────────────────────────────────────────────────
// The 256 MB memory-side cache in front of HBM keeps what was last read or written. When
// a program's recent working set is larger than that, an eager backend keeps pushing out
// data the next call wants with data nothing will touch again in time: results that are
// never read back while they are still cached (the last tensor of a chain), operands that
// are read once per pass over a long sequence. Which is which cannot be seen from one
// call, but programs repeat themselves and the allocator hands the same blocks to the
// same roles, so each large block carries a two-bit history: "what was written here was
// read again within the cache's reach", and the same for what was read. While the working
// set exceeds the cache, a block whose history says no is accessed with non-temporal loads
// or stores, which do not displace cached data; such accesses do not advance `cache_pos`,
// the measure of reach (bytes of allocating traffic issued). While everything fits,
// nothing streams: a write-back cache that absorbs a dead result still beats writing it
// to memory at once (f32 mul of two [4096,4096] operands in a loop: 7.1 TB/s with plain
// stores, 6.2 with streaming ones).
// Measured on the seven-call [64,512,512] step (496 MiB of tensors): 163 -> 142 us.
static constexpr uint64_t CACHE_REACH = (uint64_t)208 << 20;     // of the cache's 256 MB
static constexpr uint64_t CACHE_HINT_MIN = (uint64_t)8 << 20;    // smaller operands are not tracked
static constexpr uint64_t CACHE_PRESSURE = (uint64_t)232 << 20;  // working set from which blocks stream

// Bytes of the distinct blocks among the last large-operand accesses.
static uint64_t recent_working_set(const nxh_context *ctx) {
  uint64_t sum = 0;
  for (int i = 0; i < nxh_context::RECENT; i++) {
    if (!ctx->recent_block[i]) continue;
    uint64_t most = ctx->recent_bytes[i];
    bool first = true;
    for (int j = 0; j < nxh_context::RECENT; j++)
      if (j != i && ctx->recent_block[j] == ctx->recent_block[i]) {
        if (j < i) first = false;
        most = std::max(most, ctx->recent_bytes[j]);
      }
    if (first) sum += most;
  }
  return sum;
}

uint32_t nxh_cache_hints(nxh_context *ctx, int nop, const void *const *base, const uint64_t *bytes, uint32_t allow) {
  if (ctx->cache_hints & 4) {  // every access the kernels can stream does (for tests of those paths)
    ctx->streamed_in += (allow & NXH_STREAM_IN) != 0;
    ctx->streamed_out += (allow & NXH_STREAM_OUT) != 0;
    return allow;
  }
  const uint64_t pos = ctx->cache_pos;
  nxh_context::BlockUse *use[8] = {};
  if (nop > 8) nop = 8;
  // reads first: an operand that is also the output is read before it is written
  bool in_tracked = false, in_stream = true, out_stream = false;
  for (int pass = 0; pass < 2; pass++) {
    for (int k = pass == 0 ? 1 : 0; k < (pass == 0 ? nop : 1); k++) {
      const uint8_t kind = k == 0 ? 2 : 1;
      if (!ctx->cache_hints || bytes[k] < CACHE_HINT_MIN || ctx->live.find((void *)base[k]) == ctx->live.end()) continue;
      nxh_context::BlockUse &u = ctx->block_use[base[k]];
      use[k] = &u;
      ctx->recent_block[ctx->recent_next] = base[k];
      ctx->recent_bytes[ctx->recent_next] = bytes[k];
      ctx->recent_next = (ctx->recent_next + 1) % nxh_context::RECENT;
      if (u.kind && !(u.kind == 1 && kind == 1 && u.pos == pos)) {  // (not: one block read through two operands)
        const bool reused = kind == 1 && pos - u.pos <= CACHE_REACH;
        uint8_t &c = u.kind == 2 ? u.after_write : u.after_read;
        if (reused) c = (uint8_t)std::min(3, c + 1);
        else if (u.opaque == ctx->opaque_calls) c = (uint8_t)std::max(0, c - 1);  // nothing else can have read it
      }
      if (kind == 1) {
        in_tracked = true;
        if (u.after_read >= 2) in_stream = false;
      } else {
        out_stream = u.after_write < 2;
      }
      u.kind = kind;
      u.pos = pos;
      u.opaque = ctx->opaque_calls;
    }
  }
  // one decision for all inputs: they stream only if every large one is predicted to
  const bool pressure = (in_tracked || use[0]) && recent_working_set(ctx) > CACHE_PRESSURE;
  in_stream = in_stream && in_tracked && pressure && (ctx->cache_hints & 1) && (allow & NXH_STREAM_IN);
  out_stream = out_stream && pressure && (ctx->cache_hints & 2) && (allow & NXH_STREAM_OUT);
  for (int k = 0; k < nop; k++) {
    const bool streams = use[k] && (k == 0 ? out_stream : in_stream);
    if (!streams) ctx->cache_pos += bytes[k];
  }
  ctx->streamed_in += in_stream;
  ctx->streamed_out += out_stream;
  return (out_stream ? NXH_STREAM_OUT : 0u) | (in_stream ? NXH_STREAM_IN : 0u);
}

static uint64_t tensor_bytes(const nxh_tensor *t) {
  uint64_t n = 1;
  for (int d = 0; d < t->ndim && d < NXH_MAX_NDIM; d++)
    if (t->strides[d] != 0) n *= (uint64_t)(t->shape[d] < 0 ? 0 : t->shape[d]);
  return nxh_is_packed(t->dtype) ? (n + 1) / 2 : n * (uint64_t)nxh_elem_size(t->dtype);
}

void nxh_cache_touch(nxh_context *ctx, const nxh_tensor *const *tensors, int n, int n_out) {
  if (!ctx->cache_hints) return;
  // every written tensor is an access of its own; the tensors read share one
  std::lock_guard<std::mutex> g(ctx->mu);
  const void *base[8];
  uint64_t bytes[8];
  int nop = 1;
  base[0] = nullptr;
  bytes[0] = 0;
  for (int i = n_out; i < n && nop < 8; i++)
    if (tensors[i] && (unsigned)tensors[i]->ndim <= NXH_MAX_NDIM) {
      base[nop] = tensors[i]->data;
      bytes[nop++] = tensor_bytes(tensors[i]);
    }
  bool first = true;
  for (int i = 0; i < n_out || first; i++) {
    const nxh_tensor *o = i < n_out ? tensors[i] : nullptr;
    if (o && (unsigned)o->ndim > NXH_MAX_NDIM) o = nullptr;
    base[0] = o ? o->data : nullptr;
    bytes[0] = o ? tensor_bytes(o) : 0;
    (void)nxh_cache_hints(ctx, first ? nop : 1, base, bytes, 0);
    first = false;
  }
}

void nxh_cache_opaque(nxh_context *ctx) {
  std::lock_guard<std::mutex> g(ctx->mu);
  ctx->opaque_calls++;
}

NXH_EXPORT int nxh_set_cache_policy(nxh_context *ctx, int mode) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "set_cache_policy", "null context");
  if (mode < 0 || mode > 7) return nxh_fail(NXH_INVALID_ARGUMENT, "set_cache_policy", "mode must be 0..7");
  std::lock_guard<std::mutex> g(ctx->mu);
  ctx->cache_hints = mode;
  return NXH_OK;
}

NXH_EXPORT int nxh_cache_policy_stats(nxh_context *ctx, uint64_t *calls_streaming_in, uint64_t *calls_streaming_out) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "cache_policy_stats", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (calls_streaming_in) *calls_streaming_in = ctx->streamed_in;
  if (calls_streaming_out) *calls_streaming_out = ctx->streamed_out;
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
  bool recorded = false;  // deferred mode: a small upload waits in the record with its bytes
  if (int drc = nxh_defer_uploaded(ctx, dst, src, bytes, &recorded)) return drc;
  if (recorded) return NXH_OK;
  std::lock_guard<std::mutex> g(ctx->mu);
  ctx->opaque_calls++;  // writes a block that is not named to the cache policy
  NXH_HIP("from_host", hipSetDevice(ctx->device));
  if (ctx->capture) {
    // recorded as a copy from pinned memory the graph keeps: every replay uploads these bytes again
    if (bytes > nxh_context::STAGE_BYTES)
      return nxh_fail(NXH_FAILURE, "from_host", "uploads over 256 KiB are not recorded into a graph");
    void *pin = nullptr;
    NXH_HIP("from_host", hipHostMalloc(&pin, bytes, hipHostMallocDefault));
    ctx->capture->pinned.push_back(pin);
    memcpy(pin, src, bytes);
    NXH_HIP("from_host", hipMemcpyAsync(dst, pin, bytes, hipMemcpyHostToDevice, ctx->stream));
    return NXH_OK;
  }
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

// Reads the out-of-bounds flag back after a gather or scatter launch: the failure
// is reported by the call that caused it (nx_c_move.c:448-458, 571-586). A stream
// that is being recorded cannot be waited for: there the flag stays on the device
// and the next synchronize after a replay reports it.
static int read_fault_flag(nxh_context *ctx, const char *op, const char *message) {
  NXH_HIP(op, hipMemcpyAsync(ctx->fault_flag_host, ctx->fault_flag, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  NXH_HIP(op, hipStreamSynchronize(ctx->stream));
  if (*ctx->fault_flag_host == 0) return NXH_OK;
  *ctx->fault_flag_host = 0;
  NXH_HIP(op, hipMemcpyAsync(ctx->fault_flag, ctx->fault_flag_host, sizeof(int), hipMemcpyHostToDevice, ctx->stream));
  NXH_HIP(op, hipStreamSynchronize(ctx->stream));
  return nxh_fail(NXH_FAILURE, op, message);
}

int nxh_collect_index_fault(nxh_context *ctx, const char *op) {
  if (ctx->capture) {
    ctx->capture->has_index_checks = true;
    return NXH_OK;
  }
  return read_fault_flag(ctx, op, NXH_ERR_INDEX_OOB);
}

static int report_deferred_faults(nxh_context *ctx, const char *op) {
  if (!ctx->deferred_faults) return NXH_OK;
  return read_fault_flag(ctx, op, "index out of bounds in a replayed gather or scatter");
}

int nxh_settle_replay_faults(nxh_context *ctx, const char *op) {
  if (ctx->capture) return NXH_OK;
  return report_deferred_faults(ctx, op);
}

NXH_EXPORT int nxh_memcpy_d2h(nxh_context *ctx, void *dst, const void *src, size_t bytes) {
  if (ctx && nxh_defer_active(ctx))
    if (int drc = nxh_defer_host_read(ctx, src)) return drc;
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "to_host", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  ctx->opaque_calls++;  // reads a block that is not named to the cache policy
  if (int rc = refuse_while_capturing(ctx, "to_host")) return rc;
  NXH_HIP("to_host", hipSetDevice(ctx->device));
  if (bytes)
    NXH_HIP("to_host", hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  NXH_HIP("to_host", hipStreamSynchronize(ctx->stream));
  return NXH_OK;
}

NXH_EXPORT int nxh_synchronize(nxh_context *ctx) {
  NXH_DEFER_QUIET(ctx);
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "synchronize", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (int rc = refuse_while_capturing(ctx, "synchronize")) return rc;
  NXH_HIP("synchronize", hipSetDevice(ctx->device));
  NXH_HIP("synchronize", hipStreamSynchronize(ctx->stream));
  return report_deferred_faults(ctx, "synchronize");
}

// ── graphs ─────────────────────────────────────────────────────────────────
// Everything launched between capture_begin and capture_end is recorded instead
// of run. Blocks allocated in between belong to the graph until it is destroyed
// (its replays write there), including those whose tensors die during the
// capture: these are recycled inside the capture exactly as the eager allocator
// would recycle them, so a replay walks the same addresses in the same order.
// Callers hold ctx->mu and have drained the stream.
static void graph_release(nxh_context *ctx, nxh_graph *gr) {
  if (gr->exec && gr->has_index_checks) ctx->deferred_faults--;
  if (gr->exec) (void)hipGraphExecDestroy(gr->exec);
  if (gr->graph) (void)hipGraphDestroy(gr->graph);
  for (void *p : gr->pinned) (void)hipHostFree(p);
  // its idle blocks go back to the context's free lists; blocks still inside a
  // tensor become ordinary blocks
  for (auto &kv : gr->free_lists)
    for (void *p : kv.second) {
      ctx->free_lists[kv.first].push_back(p);
      ctx->cached += kv.first;
    }
  for (auto it = ctx->graph_blocks.begin(); it != ctx->graph_blocks.end();)
    it = it->second == gr ? ctx->graph_blocks.erase(it) : std::next(it);
  delete gr;
  if (--ctx->graphs_alive <= 0) {  // no record reads the GELU tables any more: they may take other constants
    ctx->graphs_alive = 0;
    ctx->gelu_lut_recorded[0] = ctx->gelu_lut_recorded[1] = false;
    ctx->gelu_epi.recorded = false;
  }
}

NXH_EXPORT int nxh_capture_begin(nxh_context *ctx) {
  NXH_DEFER_BARRIER(ctx);
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "capture_begin", "null context");
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);  // not in the middle of a factorisation
  std::lock_guard<std::mutex> g(ctx->mu);
  if (int rc = refuse_while_capturing(ctx, "capture_begin")) return rc;
  NXH_HIP("capture_begin", hipSetDevice(ctx->device));
  NXH_HIP("capture_begin", hipStreamSynchronize(ctx->stream));
  nxh_graph *gr = new nxh_graph();
  ctx->graphs_alive++;
  hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) {
    delete gr;
    ctx->graphs_alive--;
    return nxh_hip_fail("capture_begin", e);
  }
  ctx->capture = gr;
  return NXH_OK;
}

NXH_EXPORT int nxh_capture_end(nxh_context *ctx, nxh_graph **out) {
  NXH_DEFER_QUIET(ctx);
  if (!ctx || !out) return nxh_fail(NXH_INVALID_ARGUMENT, "capture_end", "null argument");
  std::lock_guard<std::mutex> g(ctx->mu);
  *out = nullptr;
  nxh_graph *gr = ctx->capture;
  if (!gr) return nxh_fail(NXH_FAILURE, "capture_end", "no capture in progress");
  ctx->capture = nullptr;
  hipError_t e = hipStreamEndCapture(ctx->stream, &gr->graph);
  if (e == hipSuccess) e = hipGraphInstantiate(&gr->exec, gr->graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    (void)hipStreamSynchronize(ctx->stream);
    graph_release(ctx, gr);
    return nxh_hip_fail("capture_end", e);
  }
  if (gr->has_index_checks) ctx->deferred_faults++;
  *out = gr;
  return NXH_OK;
}

NXH_EXPORT int nxh_graph_launch(nxh_context *ctx, nxh_graph *gr) {
  NXH_DEFER_BARRIER(ctx);
  if (!ctx || !gr || !gr->exec) return nxh_fail(NXH_INVALID_ARGUMENT, "graph_launch", "null argument");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (int rc = refuse_while_capturing(ctx, "graph_launch")) return rc;
  NXH_HIP("graph_launch", hipSetDevice(ctx->device));
  NXH_HIP("graph_launch", hipGraphLaunch(gr->exec, ctx->stream));
  return NXH_OK;
}

NXH_EXPORT int nxh_graph_destroy(nxh_context *ctx, nxh_graph *gr) {
  NXH_DEFER_QUIET(ctx);
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "graph_destroy", "null context");
  if (!gr) return NXH_OK;
  std::lock_guard<std::mutex> g(ctx->mu);
  if (ctx->capture == gr) return nxh_fail(NXH_FAILURE, "graph_destroy", "this graph is still being captured");
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  // a fault of its last replays is not lost with it
  const int rc = gr->exec && gr->has_index_checks ? report_deferred_faults(ctx, "graph_destroy") : NXH_OK;
  graph_release(ctx, gr);
  return rc;
}

// ── timing ─────────────────────────────────────────────────────────────────
NXH_EXPORT int nxh_timer_start(nxh_context *ctx) {
  NXH_DEFER_QUIET(ctx);
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "timer", "null context");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (int rc = refuse_while_capturing(ctx, "timer")) return rc;
  NXH_HIP("timer", hipEventRecord(ctx->ev_start, ctx->stream));
  return NXH_OK;
}
NXH_EXPORT int nxh_timer_stop(nxh_context *ctx, float *ms) {
  NXH_DEFER_QUIET(ctx);
  if (!ctx || !ms) return nxh_fail(NXH_INVALID_ARGUMENT, "timer", "null argument");
  std::lock_guard<std::mutex> g(ctx->mu);
  if (int rc = refuse_while_capturing(ctx, "timer")) return rc;
  NXH_HIP("timer", hipEventRecord(ctx->ev_stop, ctx->stream));
  NXH_HIP("timer", hipEventSynchronize(ctx->ev_stop));
  NXH_HIP("timer", hipEventElapsedTime(ms, ctx->ev_start, ctx->ev_stop));
  return NXH_OK;
}
