// nxh_common.hpp — shared host/device definitions of libnxhip (gfx950 only).
//
// The dtype table below is the device-side counterpart of the reference's
// single dtype table (packages/nx/lib/backend_c/nx_c.h:130-168): storage type,
// compute type, load/store converters and category per dtype. The converters
// reproduce packages/nx/lib/buffer/nx_buffer_stubs.h:70-302 bit for bit.
#pragma once

#include <algorithm>

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/nxhip.h"

#define NXH_EXPORT extern "C" __attribute__((visibility("default")))

// ─────────────────────────── context ────────────────────────────────────────

struct nxh_context {
  int device = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  int compute_units = 0;
  char name[128] = {0};
  std::mutex mu;  // guards the allocator and launches: one stream per context
  // held for the whole of a call made of several locked steps (the factorisations) and by
  // capture_begin, so that no capture starts in the middle of one; taken before `mu`
  std::mutex call_mu;
  // caching allocator: size class -> free blocks
  std::map<size_t, std::vector<void *>> free_lists;
  std::map<void *, size_t> live;  // every block handed out or cached -> its class size
  uint64_t in_use = 0, cached = 0, reserved = 0, driver_allocs = 0;
  // one device word, written by kernels that detect a data fault (gather OOB)
  int *fault_flag = nullptr;       // device
  int *fault_flag_host = nullptr;  // pinned host mirror for the readback
  // pinned staging slots for small host-to-device uploads: the caller's bytes
  // are copied into a slot and the transfer is queued on the stream, so an
  // upload does not wait for the work already queued
  static constexpr int STAGE_SLOTS = 16;
  static constexpr size_t STAGE_BYTES = (size_t)256 << 10;
  char *stage = nullptr;  // STAGE_SLOTS * STAGE_BYTES
  hipEvent_t stage_done[STAGE_SLOTS] = {};
  bool stage_used[STAGE_SLOTS] = {};
  int stage_next = 0;
  // stream capture: while `capture` is set, launches are recorded into its graph
  // and allocations come from (and go back to) the graph's own blocks
  struct nxh_graph *capture = nullptr;
  std::map<void *, struct nxh_graph *> graph_blocks;  // block -> the graph that holds it
  // twiddle and chirp tables of the transforms, by (kind, sign, length); freed with the context
  std::map<uint64_t, void *> device_tables;
  int deferred_faults = 0;  // live graphs whose gathers / scatters report at the next synchronize
  // this device's copy of the library's static workspace (runtime.hip), for the
  // entry point that may not allocate; shared by every context of the device
  unsigned char *static_ws = nullptr;
  // Reuse predictor for the 256 MB memory-side cache (runtime.hip, nxh_cache_hints): per
  // block of 8 MiB or more, where the stream of cache-allocating traffic stood at its
  // last access, what that access was, and two 2-bit counters: was the block read again
  // while it could still be cached, after a write and after a read.
  struct BlockUse {
    uint64_t pos = 0;
    uint8_t kind = 0;          // 0 never seen, 1 read, 2 written
    uint8_t after_write = 2;   // >= 2: keep what is written here in the cache
    uint8_t after_read = 2;    // >= 2: keep what is read from here in the cache
    uint64_t opaque = 0;       // opaque_calls at that access
  };
  std::unordered_map<const void *, BlockUse> block_use;
  uint64_t cache_pos = 0;  // bytes of cache-allocating traffic issued so far
  // the last large-operand accesses (block, bytes): their distinct blocks are the working set
  static constexpr int RECENT = 32;
  const void *recent_block[RECENT] = {};
  uint64_t recent_bytes[RECENT] = {};
  int recent_next = 0;
  int cache_hints = 3;     // bit 0: streaming loads allowed, bit 1: streaming stores (NXH_CACHE_HINTS)
  uint64_t streamed_in = 0, streamed_out = 0;  // calls whose inputs / result streamed
  // calls so far that may have read or written any block without saying which (transforms,
  // factorisations, sorts, graph replays, host copies): no block counts as "not touched
  // again" across one of them
  uint64_t opaque_calls = 0;
  // State of the single-pass column scan (scan.hip, scan_cols): a device block holding one
  // 64-bit (flag, value) word per column and row chunk; flags carry the launch's epoch, so the words are cleared once, when the block is
  // made, and never between launches. Freed with the context.
  // results of the tanh GELU for all 65 536 inputs of bf16 [0] and f16 [1] (rowfuse.hip), and the
  // four constants each table was made with
  void *gelu_lut[2] = {nullptr, nullptr};
  double gelu_lut_c[2][4] = {};
  // a recorded graph reads the table: it keeps its constants from then on (other constants take the arithmetic)
  bool gelu_lut_recorded[2] = {false, false};
  int graphs_alive = 0;  // recorded graphs not yet destroyed (the one being captured included)
  // The part of the bfloat16 table the fused linear's GELU epilogue keeps in LDS (rowfuse.hip,
  // nxh_gelu_epilogue_table): entries [lo, lo + n) of either sign, n*2 values on the device;
  // state 0 not made yet, 1 usable, -1 these constants have no usable form.
  struct GeluEpilogueTable {
    int state = 0;
    double c[4] = {};
    uint32_t lo = 0, n = 0;
    void *dev = nullptr;
    bool recorded = false;  // a recorded graph reads dev: its contents stay
  } gelu_epi;
  unsigned char *scan_state = nullptr;
  size_t scan_state_bytes = 0;
  uint32_t scan_epoch = 0;
};

// bfloat16 only. On success *table is a device array of 2 * *n results (the non-negative
// inputs with magnitude bits [lo, lo + n), then the negative ones) of the tanh GELU with the
// constants c; 0 when there is none (being made would need to wait for the stream, which a
// capture forbids, or the constants do not fit the scheme). Called with ctx->mu held.
int nxh_gelu_epilogue_table(nxh_context *ctx, const double *c, const void **table, uint32_t *lo, uint32_t *n);

// Size of the static per-device workspace behind nxh_reduce_noalloc.
constexpr size_t NXH_STATIC_WS_BYTES = (size_t)NXH_STATIC_WORKSPACE_BYTES;

// A captured sequence of launches (runtime.hip).
struct nxh_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::map<size_t, std::vector<void *>> free_lists;  // its blocks not in use by a tensor
  std::vector<void *> pinned;                        // host staging of captured uploads
  bool has_index_checks = false;
};

// thread-local status text (static strings + op prefix)
void nxh_set_error(const char *op, const char *msg);
void nxh_set_path(const char *path);
int nxh_fail(int kind, const char *op, const char *msg);
int nxh_hip_fail(const char *op, hipError_t e);

#define NXH_HIP(op, call)                                \
  do {                                                   \
    hipError_t e__ = (call);                             \
    if (e__ != hipSuccess) return nxh_hip_fail(op, e__); \
  } while (0)

// allocator (runtime.hip)
int nxh_alloc_locked(nxh_context *ctx, size_t bytes, void **out);
void nxh_free_locked(nxh_context *ctx, void *p);
// Cache hints of one launch (runtime.hip). Operand 0 is written, the others are read;
// `base` are the tensors' data pointers (block bases), `bytes` the distinct bytes the launch
// touches of each. Returns NXH_STREAM_OUT if what is written should go past the memory-side
// cache (non-temporal stores) and NXH_STREAM_IN if what is read should (non-temporal loads of
// every large input). Caller holds ctx->mu.
enum { NXH_STREAM_OUT = 1u, NXH_STREAM_IN = 2u };
uint32_t nxh_cache_hints(nxh_context *ctx, int nop, const void *const *base, const uint64_t *bytes,
                         uint32_t allow = NXH_STREAM_OUT | NXH_STREAM_IN);
// The same bookkeeping for an entry point whose kernels take no hints: the first n_out
// tensors are written, the others read (NULL entries are skipped). Takes ctx->mu.
void nxh_cache_touch(nxh_context *ctx, const nxh_tensor *const *tensors, int n, int n_out);
// An entry point that may touch blocks it does not name. Takes ctx->mu.
void nxh_cache_opaque(nxh_context *ctx);
// the out-of-bounds flag of gather / scatter, read back (or left for the replay) (runtime.hip)
int nxh_collect_index_fault(nxh_context *ctx, const char *op);
// Before an eager gather / scatter is launched: a fault that a replayed graph left in
// the flag is reported now, as the replay's, so that this call answers only for itself.
int nxh_settle_replay_faults(nxh_context *ctx, const char *op);

// several linear layers over one x as one launch (matmul.hip); used by the deferred window
int nxh_linear_group(nxh_context *ctx, int n, const nxh_tensor *const *outs, const nxh_tensor *x,
                     const nxh_tensor *const *ws, const nxh_tensor *const *biases);
// the deferred-evaluation window (defer.hip)
bool nxh_defer_active(nxh_context *ctx);
int nxh_defer_flush(nxh_context *ctx);
int nxh_defer_barrier(nxh_context *ctx, const nxh_tensor *out0 = nullptr, const nxh_tensor *out1 = nullptr,
                      const nxh_tensor *out2 = nullptr);
int nxh_defer_touch(nxh_context *ctx, const nxh_tensor *const *tensors, int n, int n_out);
int nxh_defer_quiet(nxh_context *ctx);
int nxh_defer_host_read(nxh_context *ctx, const void *src);
int nxh_defer_record(nxh_context *ctx, int kind, int op, const nxh_tensor *out, const nxh_tensor *const *ins, int nin,
                     const int32_t *axes, int n_axes, const void *value);
bool nxh_defer_free(nxh_context *ctx, void *p);
int nxh_defer_uploaded(nxh_context *ctx, void *dst, const void *src, size_t bytes, bool *recorded);
void nxh_defer_context_gone(nxh_context *ctx);
enum { NXH_D_UNARY, NXH_D_BINARY, NXH_D_COMPARE, NXH_D_WHERE, NXH_D_CAST, NXH_D_REDUCE, NXH_D_MATMUL, NXH_D_FULL, NXH_D_COPY, NXH_D_UPLOAD };
// Entry points that are not recorded run the record first. BARRIER also writes everything
// that was postponed; TOUCH (the first n_out tensors are written, the others read; NULL entries
// are skipped) only what those blocks need; QUIET nothing.
#define NXH_DEFER_BARRIER(ctx, ...)                              \
  do {                                                           \
    if ((ctx) && nxh_defer_active(ctx))                          \
      if (int drc__ = nxh_defer_barrier(ctx, ##__VA_ARGS__)) return drc__; \
    if (ctx) nxh_cache_opaque(ctx);                              \
  } while (0)
#define NXH_DEFER_TOUCH(ctx, n_out, ...)                                                                      \
  do {                                                                                                        \
    if (ctx) {                                                                                                \
      const nxh_tensor *dts__[] = {__VA_ARGS__};                                                              \
      if (nxh_defer_active(ctx))                                                                              \
        if (int drc__ = nxh_defer_touch(ctx, dts__, (int)(sizeof dts__ / sizeof *dts__), n_out)) return drc__; \
      nxh_cache_touch(ctx, dts__, (int)(sizeof dts__ / sizeof *dts__), n_out);                                \
    }                                                                                                         \
  } while (0)
// As TOUCH, for entry points that ask nxh_cache_hints themselves (once their arguments are checked).
#define NXH_DEFER_SETTLE(ctx, n_out, ...)                                                                     \
  do {                                                                                                        \
    if ((ctx) && nxh_defer_active(ctx)) {                                                                     \
      const nxh_tensor *dts__[] = {__VA_ARGS__};                                                              \
      if (int drc__ = nxh_defer_touch(ctx, dts__, (int)(sizeof dts__ / sizeof *dts__), n_out)) return drc__; \
    }                                                                                                         \
  } while (0)
#define NXH_DEFER_QUIET(ctx)                                     \
  do {                                                           \
    if ((ctx) && nxh_defer_active(ctx))                          \
      if (int drc__ = nxh_defer_quiet(ctx)) return drc__;        \
  } while (0)
// Recorded entry points: NXH_OK means recorded; -1 means run now.
#define NXH_DEFER_RECORD(ctx, kind, op, out, nin, axes, n_axes, value, ...)                             \
  do {                                                                                                  \
    if ((ctx) && nxh_defer_active(ctx)) {                                                               \
      const nxh_tensor *dins__[] = {__VA_ARGS__};                                                       \
      const int drc__ = nxh_defer_record(ctx, kind, op, out, dins__, nin, axes, n_axes, value);         \
      if (drc__ != -1) return drc__;                                                                    \
    }                                                                                                   \
  } while (0)

// status strings shared with the reference (nx_c.h:381-388, nx_c_engine.h:38-50)
#define NXH_ERR_NDIM "ndim exceeds NX_C_MAX_NDIM"
#define NXH_ERR_BAD_KIND "unsupported bigarray kind"
#define NXH_ERR_UNSUPPORTED "dtype not supported for this operation"
#define NXH_ERR_PACKED "packed dtype not supported for this operation"
#define NXH_ERR_SHAPE "shape mismatch"
#define NXH_ERR_EMPTY_REDUCE "reduction over empty axis has no identity"
#define NXH_ERR_ALLOC "out of memory"
#define NXH_ERR_AXES "reduce axes must be strictly increasing and in range"
#define NXH_ERR_OUT_RANK "output rank inconsistent with the operation"
#define NXH_ERR_AXIS "axis out of range"
#define NXH_ERR_OUT_ALIASED "output has a broadcast (zero) stride"
#define NXH_ERR_ARGCAP "argreduce axis length exceeds INT32_MAX"
#define NXH_ERR_INDEX_OOB "index out of bounds for the gathered/scattered axis"
#define NXH_ERR_MM_DTYPE "matmul operands must share one dtype"

static inline bool nxh_is_packed(int dt) { return dt == NXH_I4 || dt == NXH_U4; }
static inline int64_t nxh_elem_size(int dt) {
  static const int64_t s[NXH_DTYPE_COUNT] = {2, 4, 8, 2, 1, 1, 0, 0, 1, 1,
                                             2, 2, 4, 4, 8, 8, 8, 16, 1};
  return (unsigned)dt < NXH_DTYPE_COUNT ? s[dt] : 0;
}
static inline bool nxh_same_shape(const nxh_tensor *a, const nxh_tensor *b) {
  if (a->ndim != b->ndim) return false;
  for (int i = 0; i < a->ndim; i++)
    if (a->shape[i] != b->shape[i]) return false;
  return true;
}
static inline int nxh_check_tensor(const char *op, const nxh_tensor *t) {
  if (t->ndim < 0 || t->ndim > NXH_MAX_NDIM) return nxh_fail(NXH_FAILURE, op, NXH_ERR_NDIM);
  if ((unsigned)t->dtype >= NXH_DTYPE_COUNT) return nxh_fail(NXH_FAILURE, op, NXH_ERR_BAD_KIND);
  return NXH_OK;
}

// ─────────────────────────── device scalar types ────────────────────────────

enum Cat { CAT_SINT, CAT_UINT, CAT_FLOAT, CAT_COMPLEX, CAT_BOOL };

template <class R>
struct cplx {
  R re, im;
};
using c32 = cplx<float>;
using c64 = cplx<double>;

#define HD __host__ __device__ __forceinline__

template <class R>
HD cplx<R> operator+(cplx<R> a, cplx<R> b) { return {a.re + b.re, a.im + b.im}; }
template <class R>
HD cplx<R> operator-(cplx<R> a, cplx<R> b) { return {a.re - b.re, a.im - b.im}; }
template <class R>
HD cplx<R> operator-(cplx<R> a) { return {-a.re, -a.im}; }
template <class R>
HD cplx<R> operator*(cplx<R> a, cplx<R> b) {
  return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
// Smith's division: no intermediate overflow for representable quotients.
template <class R>
HD cplx<R> operator/(cplx<R> a, cplx<R> b) {
  if (fabs(b.re) >= fabs(b.im)) {
    if (b.re == 0 && b.im == 0) return {a.re / b.re, a.im / b.re};
    R r = b.im / b.re, d = b.re + b.im * r;
    return {(a.re + a.im * r) / d, (a.im - a.re * r) / d};
  }
  R r = b.re / b.im, d = b.re * r + b.im;
  return {(a.re * r + a.im) / d, (a.im * r - a.re) / d};
}
template <class R>
HD bool operator==(cplx<R> a, cplx<R> b) { return a.re == b.re && a.im == b.im; }
template <class R>
HD bool operator!=(cplx<R> a, cplx<R> b) { return !(a == b); }

HD uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
HD float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// f32 -> bf16, nx_buffer_stubs.h:73-86: NaN keeps sign/payload and is quieted,
// everything else rounds to nearest even on the dropped half.
HD uint16_t f32_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  // One v_cvt_pk_bf16_f32. It returns what the rule below returns for every one of
  // the 2^32 float bit patterns, NaNs included (compared exhaustively on an MI355X);
  // the rule itself costs eight integer instructions per element, which made the
  // narrowing epilogues and the fused row kernels VALU-bound.
  // The barrier keeps the conversion a scalar one: without it the compiler pairs it
  // with neighbouring float operations into two-element vector nodes that the
  // backend cannot select when packed f32 operations are switched off.
  asm("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, (__bf16)f);
#else
  uint32_t u = f2u(f);
  uint32_t nan = (u >> 16) | 0x40u;
  uint32_t rne = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return (uint16_t)(((u & 0x7fffffffu) > 0x7f800000u) ? nan : rne);
#endif
}
HD float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
// Two neighbours narrowed by ONE v_cvt_pk_bf16_f32: `lo` in the low half.
HD uint32_t f32x2_to_bf16x2(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  asm("" : "+v"(lo), "+v"(hi));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
#else
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
#endif
}

// tanh for a result that is rounded to a 16-bit float right behind it (bfloat16 / float16
// tensors compute in float): (1 - t) / (1 + t) with t = e^(-2|x|) from the hardware
// exponential and reciprocal, the odd polynomial x - x^3/3 + 2x^5/15 - 17x^7/315 below 1/8
// where that quotient cancels. Within 4e-7 relative of tanh, against the 2^-12 of a float16
// rounding; the library's tanhf costs about four times as many instructions and made the
// fused GELU and the tanh primitive of those dtypes bound by the vector unit. NaN stays NaN,
// the sign of zero is kept, +-inf gives +-1.
__device__ __forceinline__ float tanh_for_16bit(float x) {
  const float ax = __builtin_fabsf(x);
  const float t = __builtin_amdgcn_exp2f(ax * -0x1.715476p+1f);  // e^(-2|x|)
  const float big = (1.0f - t) * __builtin_amdgcn_rcpf(1.0f + t);
  const float x2 = x * x;
  const float small = ax * __builtin_fmaf(x2, __builtin_fmaf(x2, __builtin_fmaf(x2, -0x1.ba1ba2p-5f, 0x1.111112p-3f), -0x1.555556p-2f), 1.0f);
  return __builtin_copysignf(ax < 0.125f ? small : big, x);
}
// f32 -> f16, nx_buffer_stubs.h:99-148. The hardware convert (round to nearest
// even, subnormals kept) matches on every non-NaN input; a NaN keeps its top
// ten payload bits and is bumped to stay a NaN.
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  // Keep the narrowing a plain v_cvt_f16_f32. Without the barrier the compiler
  // folds a preceding multiply into v_fma_mixlo_f16(a, b, +0), and (-0) + (+0)
  // turns a negative-zero product into +0.
  asm("" : "+v"(f));
  uint32_t u = f2u(f);
  _Float16 h = (_Float16)f;
  uint16_t hw = __builtin_bit_cast(uint16_t, h);
  uint32_t m = u & 0x7fffffu;
  uint32_t r = 0x7c00u + (m >> 13);
  r += (r == 0x7c00u);
  uint16_t nan = (uint16_t)(((u >> 16) & 0x8000u) + r);
  return ((u & 0x7fffffffu) > 0x7f800000u) ? nan : hw;
}
// f16 -> f32, nx_buffer_stubs.h:150-182: exact; NaN payload shifts up and the
// quiet bit is forced.
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  _Float16 x = __builtin_bit_cast(_Float16, h);
  float hw = (float)x;
  uint32_t nan = (((uint32_t)h & 0x8000u) << 16) | 0x7f800000u | (((uint32_t)h & 0x3ffu) << 13) |
                 0x400000u;
  return ((h & 0x7fffu) > 0x7c00u) ? u2f(nan) : hw;
}

// Shared fp8 encoder body (nx_buffer_stubs.h:189-223, 244-278).
template <int MBITS, int BIAS>
HD uint32_t f32_to_fp8_bits(uint32_t u) {
  int exp = (int)((u >> 23) & 0xffu) - 127;
  constexpr int EMIN = 1 - BIAS;
  if (exp >= EMIN) {
    uint32_t sig = u & 0x7fffffu;
    constexpr int drop = 23 - MBITS;
    uint32_t q = sig >> drop, rem = sig & ((1u << drop) - 1u), half = 1u << (drop - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return ((uint32_t)(exp + BIAS) << MBITS) + q;
  }
  uint32_t sig = (u & 0x7fffffu) | 0x800000u;
  int shift = (23 - MBITS) + (EMIN - exp);
  if (shift > 24) return 0;
  uint32_t q = sig >> shift, rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return q;
}
HD uint8_t f32_to_f8e4m3(float f) {
  uint32_t u = f2u(f);
  uint32_t a = u & 0x7fffffffu;
  uint8_t sign = (uint8_t)((u >> 31) << 7);
  if (a > 0x7f800000u) return 0x7f;           // NaN: sign dropped
  if (a == 0x7f800000u) return sign | 0x7f;   // inf -> NaN, sign kept
  uint32_t bits = f32_to_fp8_bits<3, 7>(u);
  return bits >= 0x7fu ? (uint8_t)(sign | 0x7f) : (uint8_t)(sign | bits);
}
HD uint8_t f32_to_f8e5m2(float f) {
  uint32_t u = f2u(f);
  uint32_t a = u & 0x7fffffffu;
  uint8_t sign = (uint8_t)((u >> 31) << 7);
  if (a > 0x7f800000u) return 0x7f;
  if (a == 0x7f800000u) return sign | 0x7c;
  uint32_t bits = f32_to_fp8_bits<2, 15>(u);
  return bits >= 0x7cu ? (uint8_t)(sign | 0x7c) : (uint8_t)(sign | bits);
}
// Decoders (nx_buffer_stubs.h:225-240, 280-302), by exact bit construction:
// a subnormal m * 2^(emin - mbits) is built as an integer-to-float conversion
// scaled by a power of two, both exact.
HD float f8e4m3_to_f32(uint8_t v) {
  uint32_t e = (v >> 3) & 0xfu, m = v & 7u;
  if (e == 0xfu && m == 7u) return u2f(0x7fc00000u);  // NAN macro: positive quiet NaN
  float r = e == 0 ? (float)m * 0.001953125f /* 2^-9 */
                   : u2f(((e + 120u) << 23) | (m << 20));
  return (v & 0x80) ? -r : r;
}
HD float f8e5m2_to_f32(uint8_t v) {
  uint32_t e = (v >> 2) & 0x1fu, m = v & 3u;
  bool neg = (v & 0x80) != 0;
  if (e == 0x1fu) return m == 0 ? u2f(neg ? 0xff800000u : 0x7f800000u) : u2f(0x7fc00000u);
  float r = e == 0 ? (float)m * 0.0000152587890625f /* 2^-16 */
                   : u2f(((e + 112u) << 23) | (m << 21));
  return neg ? -r : r;
}

// The dtype table.
template <int DT>
struct Tr;
#define NXH_TR(DT, S_, C_, CAT_, LD_, ST_)                                \
  template <>                                                             \
  struct Tr<DT> {                                                         \
    using S = S_;                                                         \
    using C = C_;                                                         \
    static constexpr Cat cat = CAT_;                                      \
    static constexpr int tag = DT;                                        \
    __device__ __forceinline__ static C ld(S s) { return (C)(LD_(s)); }   \
    __device__ __forceinline__ static S st(C c) { return (S)(ST_(c)); }   \
  };
#define NXH_ID(x) (x)
#define NXH_BOOLN(x) ((x) != 0)
NXH_TR(NXH_F16, uint16_t, float, CAT_FLOAT, f16_to_f32, f32_to_f16)
NXH_TR(NXH_F32, float, float, CAT_FLOAT, NXH_ID, NXH_ID)
NXH_TR(NXH_F64, double, double, CAT_FLOAT, NXH_ID, NXH_ID)
NXH_TR(NXH_BF16, uint16_t, float, CAT_FLOAT, bf16_to_f32, f32_to_bf16)
NXH_TR(NXH_F8E4M3, uint8_t, float, CAT_FLOAT, f8e4m3_to_f32, f32_to_f8e4m3)
NXH_TR(NXH_F8E5M2, uint8_t, float, CAT_FLOAT, f8e5m2_to_f32, f32_to_f8e5m2)
NXH_TR(NXH_I8, int8_t, int64_t, CAT_SINT, NXH_ID, NXH_ID)
NXH_TR(NXH_U8, uint8_t, int64_t, CAT_UINT, NXH_ID, NXH_ID)
NXH_TR(NXH_I16, int16_t, int64_t, CAT_SINT, NXH_ID, NXH_ID)
NXH_TR(NXH_U16, uint16_t, int64_t, CAT_UINT, NXH_ID, NXH_ID)
NXH_TR(NXH_I32, int32_t, int64_t, CAT_SINT, NXH_ID, NXH_ID)
NXH_TR(NXH_U32, uint32_t, uint64_t, CAT_UINT, NXH_ID, NXH_ID)
NXH_TR(NXH_I64, int64_t, int64_t, CAT_SINT, NXH_ID, NXH_ID)
NXH_TR(NXH_U64, uint64_t, uint64_t, CAT_UINT, NXH_ID, NXH_ID)
NXH_TR(NXH_C32, c32, c32, CAT_COMPLEX, NXH_ID, NXH_ID)
NXH_TR(NXH_C64, c64, c64, CAT_COMPLEX, NXH_ID, NXH_ID)
NXH_TR(NXH_BOOL, uint8_t, uint8_t, CAT_BOOL, NXH_BOOLN, NXH_BOOLN)

// Applies X(DT) to every compute dtype tag (packed int4/uint4 excluded).
#define NXH_FOR_COMPUTE_DTYPES(X)                                                  \
  X(NXH_F16) X(NXH_F32) X(NXH_F64) X(NXH_BF16) X(NXH_F8E4M3) X(NXH_F8E5M2) X(NXH_I8) \
  X(NXH_U8) X(NXH_I16) X(NXH_U16) X(NXH_I32) X(NXH_U32) X(NXH_I64) X(NXH_U64)      \
  X(NXH_C32) X(NXH_C64) X(NXH_BOOL)

// Saturating double -> integer storage (nx_c.h:234-250): NaN -> 0, clamp.
template <class S>
__device__ __forceinline__ S f2i_sat(double v) {
  constexpr int w = (int)sizeof(S) * 8;
  if constexpr (std::is_signed<S>::value) {
    const double lim = (double)((uint64_t)1 << (w - 1));
    if (v != v) return 0;
    if (v <= -lim) return (S)((uint64_t)1 << (w - 1));
    if (v >= lim) return (S)(((uint64_t)1 << (w - 1)) - 1);
    return (S)(int64_t)v;
  } else {
    const double lim = w == 64 ? 18446744073709551616.0 : (double)((uint64_t)1 << (w & 63));
    if (v != v) return 0;
    if (v <= 0.0) return 0;
    if (v >= lim) return (S)(~(uint64_t)0);
    return (S)(uint64_t)v;
  }
}

// Blocks that split a strided walk (reduced rows, K-chunks of a GEMV) start
// `chunk` rows apart. When that distance is a multiple of 1 MiB every block's
// stream lands on the same few HBM channels (measured: 67% instead of 85% of
// peak on [8192, 8192] f32 with 128-row chunks), so such chunks are stretched
// by a quarter MiB of rows.
static inline int64_t chunk_off_channel_stride(int64_t chunk, int64_t row_stride_bytes) {
  const int64_t sb = row_stride_bytes < 0 ? -row_stride_bytes : row_stride_bytes;
  if (sb == 0 || (chunk * sb) % ((int64_t)1 << 20) != 0) return chunk;
  return chunk + std::max<int64_t>(1, ((int64_t)256 << 10) / sb);
}
