// fft.hip — fft / ifft / rfft / irfft (packages/nx/lib/backend_c/nx_c_fft.c).
//
// Contract kept from the reference (nx_c_fft.c:30-32, 940-1144): transforms are
// UNNORMALISED (fft is the -sign DFT, ifft the +sign DFT without 1/n); all
// arithmetic is double precision, complex64 upcasts on load and rounds once on
// store; several axes are repeated 1-D passes in the order given, the first
// reading the input, the later ones transforming the output in place; rfft is
// the full transform of the real line keeping n/2+1 bins along the LAST listed
// axis, which is transformed first; irfft transforms the other axes first (in a
// complex128 temporary), then rebuilds the length-s spectrum of the last axis by
// conjugate symmetry (zero-padding or truncating the supplied half) and keeps
// the real part of its +sign transform.
//
// How it runs here: one axis pass = one launch in which a workgroup owns one
// line (or several short ones), loads it strided into LDS as double2, does all
// radix-2 stages there (four at a time, sixteen elements per lane in registers) and stores it strided, so a pass reads and writes the
// tensor exactly once. Lengths that are not a power of two go through Bluestein's
// identity inside the same kernel: chirp on load, a power-of-two convolution of
// length M >= 2n-1 (forward DIF, multiply by the transformed chirp filter in
// bit-reversed order, inverse DIT: no reordering pass), chirp on store.
// Transforms longer than the LDS holds (power of two above 8192, other lengths
// above 4096) are staged through a complex128 workspace and done as a four-step
// (n = n1 x n2) pair of passes of the same kernel.
//
// Twiddles, chirps and chirp-filter spectra are built on the device with
// sincospi on exactly reduced arguments, once per (length, sign) and context,
// and kept until the context is destroyed (the reference's plan cache,
// nx_c_fft.c:34-44).

#include "nxh_common.hpp"

namespace {

constexpr int FFT_MAXD = 8;         // other dims of a tensor's lines after merging
constexpr int FFT_LDS_MAX = 8192;   // longest transform held in one workgroup's LDS (128 KiB)
constexpr int FFT_LDS_MIN = 2048;   // LDS elements of a workgroup of short lines
constexpr int64_t FFT_WORK_ELEMS = int64_t(1) << 25;  // workspace elements per chunk of lines (512 MiB)

enum Kind { K_C32 = 0, K_C64 = 1, K_F32 = 2, K_F64 = 3 };
enum LoadMode { LOAD_COMPLEX = 0, LOAD_REAL = 1, LOAD_HERMITIAN = 2 };

static inline int kind_size(int k) { return k == K_C32 ? 8 : k == K_C64 ? 16 : k == K_F32 ? 4 : 8; }

// Every line of a tensor along one axis: line l is decoded over `dims`
// (row-major) into an element offset, element j of it is `estride` further each.
struct Lines {
  char *base;
  int kind, nd;
  int64_t dims[FFT_MAXD], strides[FFT_MAXD];
  int64_t estride;
};

struct FftArgs {
  Lines in, out;
  int64_t lines, line0;  // lines in total; first line of this launch (workspace passes address from line0)
  int n;                 // transform length
  int M, logM;           // LDS transform length: n, or the Bluestein convolution length
  int n_load, load_mode, herm_s;
  int n_store;
  int sign;              // -1 forward, +1 inverse
  int G;                 // lines per workgroup
  // The workgroup's G lines are neighbours in memory while a line's own elements are strided
  // (a transform down the columns of a row-major tensor): consecutive lanes then take the
  // same element of consecutive lines, so that a wave's accesses are contiguous runs of G
  // elements instead of 64 separate ones. Separately for the load and the store side.
  int in_lines_fast, out_lines_fast;
  const double2 *tw;     // exp(-2 pi i k / M), k < M/2
  const double2 *chirp;  // Bluestein: exp(sign pi i j^2 / n), j < n
  const double2 *bf;     // Bluestein: forward transform (length M) of the wrapped conjugate chirp
  int64_t tw_total;      // four-step: multiply bin k of a line by exp(sign 2 pi i inner k / tw_total)
};

// Element i of the lines lives at LDS index i + i / 16: one pad element per 16
// (per 256 bytes, the width of the banks) turns the power-of-two strides of the
// butterflies and of the bit-reversed scatter into conflict-free ones.
__device__ __forceinline__ int pad(int i) { return i + (i >> 4); }

__device__ __forceinline__ double2 cmul(double2 a, double2 b) {
  return make_double2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x);
}

__device__ __forceinline__ double2 load_elem(const char *base, int kind, int64_t off) {
  switch (kind) {
    case K_C32: { const float2 v = *(const float2 *)(base + off * 8); return make_double2(v.x, v.y); }
    case K_C64: return *(const double2 *)(base + off * 16);
    case K_F32: return make_double2(*(const float *)(base + off * 4), 0.0);
    default: return make_double2(*(const double *)(base + off * 8), 0.0);
  }
}

__device__ __forceinline__ void store_elem(char *base, int kind, int64_t off, double2 v) {
  switch (kind) {
    case K_C32: *(float2 *)(base + off * 8) = make_float2((float)v.x, (float)v.y); break;
    case K_C64: *(double2 *)(base + off * 16) = v; break;
    case K_F32: *(float *)(base + off * 4) = (float)v.x; break;
    default: *(double *)(base + off * 8) = v.x; break;
  }
}

__device__ __forceinline__ int64_t line_offset(const Lines &v, int64_t l, int *inner) {
  int64_t off = 0;
  *inner = 0;
  for (int d = v.nd - 1; d >= 0; d--) {
    const int64_t c = l % v.dims[d];
    l /= v.dims[d];
    if (d == v.nd - 1) *inner = (int)c;
    off += c * v.strides[d];
  }
  return off;
}

// Element j (< n) of the sequence the transform sees, from the stored line.
__device__ __forceinline__ double2 fetch(const FftArgs &a, int64_t off, int j) {
  if (a.load_mode == LOAD_HERMITIAN) {  // nx_c_fft.c:1013-1023
    if (j < a.n_load) return load_elem(a.in.base, a.in.kind, off + j * a.in.estride);
    const int k = a.herm_s - j;
    if (k < a.n_load) {
      const double2 v = load_elem(a.in.base, a.in.kind, off + k * a.in.estride);
      return make_double2(v.x, -v.y);
    }
    return make_double2(0.0, 0.0);
  }
  if (j >= a.n_load) return make_double2(0.0, 0.0);
  return load_elem(a.in.base, a.in.kind, off + j * a.in.estride);
}

// R consecutive radix-2 stages, s .. s + R - 1 (stage s has sub-transform length
// 2^s), in one pass over the G lines of the workgroup: a lane holds the 2^R
// elements h = 2^(s-1) apart in registers and does every butterfly among them,
// so the lines go through LDS once per R stages (the stages are bound by LDS
// bandwidth: 32 bytes per element and pass). The arithmetic per element is that
// of R single stages in the same order. DIT (stages upwards): input bit-reversed,
// output natural. DIF (stages downwards): input natural, output bit-reversed.
// The twiddle table stays in global memory (small and cache-resident; a copy in
// LDS measured slower).
template <bool DIF, int R>
__device__ __forceinline__ void stages(double2 *lds, const FftArgs &a, int s, int sign) {
  constexpr int N = 1 << R;
  const double2 *tw = a.tw;
  const int h = 1 << (s - 1);
  const int per_line = a.M >> R;
  const int total = a.G * per_line;
  for (int b = threadIdx.x; b < total; b += blockDim.x) {
    const int g = b >> (a.logM - R);
    const int r = b & (per_line - 1);
    const int pos = r & (h - 1);
    const int i0 = (g << a.logM) + ((r >> (s - 1)) << (s - 1 + R)) + pos;
    double2 x[N];
#pragma unroll
    for (int k = 0; k < N; k++) x[k] = lds[pad(i0 + k * h)];
#pragma unroll
    for (int qq = 0; qq < R; qq++) {
      const int q = DIF ? R - 1 - qq : qq, span = 1 << q;
#pragma unroll
      for (int k = 0; k < N; k++) {
        if (k & span) continue;
        // the pair's position inside its sub-transform of length 2^(s+q)
        double2 w = tw[(pos + (k & (span - 1)) * h) << (a.logM - s - q)];
        if (sign > 0) w.y = -w.y;
        const double2 u = x[k], v = x[k + span];
        if (DIF) {
          x[k] = make_double2(u.x + v.x, u.y + v.y);
          x[k + span] = cmul(make_double2(u.x - v.x, u.y - v.y), w);
        } else {
          const double2 t = cmul(w, v);
          x[k] = make_double2(u.x + t.x, u.y + t.y);
          x[k + span] = make_double2(u.x - t.x, u.y - t.y);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < N; k++) lds[pad(i0 + k * h)] = x[k];
  }
  __syncthreads();
}

// All stages of the lines in LDS, FFT_RADIX_LOG2 at a time; the stages left over
// (fewer than that) go first in DIT order, last in DIF order.
constexpr int FFT_RADIX_LOG2 = 4;
template <bool DIF>
__device__ __forceinline__ void all_stages(double2 *lds, const FftArgs &a, int sign) {
  constexpr int R = FFT_RADIX_LOG2;
  const int rem = a.logM % R;
  auto odd = [&](int s) {
    if (rem == 1) stages<DIF, 1>(lds, a, s, sign);
    else if (rem == 2) stages<DIF, 2>(lds, a, s, sign);
    else if (rem == 3) stages<DIF, 3>(lds, a, s, sign);
  };
  if (DIF) {
    for (int s = a.logM - R + 1; s >= rem + 1; s -= R) stages<true, R>(lds, a, s, sign);
    odd(1);
  } else {
    odd(1);
    for (int s = rem + 1; s + R - 1 <= a.logM; s += R) stages<false, R>(lds, a, s, sign);
  }
}

template <bool BLUE>
__global__ __launch_bounds__(1024) void fft_lines_kernel(FftArgs a) {
  extern __shared__ double2 lds[];
  int64_t *off_in = (int64_t *)(lds + pad(a.G << a.logM) + 1);
  int64_t *off_out = off_in + a.G;
  int *inner = (int *)(off_out + a.G);
  // blocks that share an XCD (ids equal modulo 8) take neighbouring groups of lines: with
  // strided lines a 128-byte line of memory serves several workgroups, which then meet in one L2
  uint32_t bx = blockIdx.x;
  if ((gridDim.x & 7u) == 0) bx = (bx & 7u) * (gridDim.x >> 3) + (bx >> 3);
  const int64_t first = (int64_t)bx * a.G;
  for (int g = threadIdx.x; g < a.G; g += blockDim.x) {
    const int64_t l = first + g;
    int in_c = 0, out_c = 0;
    off_in[g] = l < a.lines ? line_offset(a.in, a.line0 + l, &in_c) : 0;
    off_out[g] = l < a.lines ? line_offset(a.out, a.line0 + l, &out_c) : 0;
    inner[g] = out_c;
  }
  __syncthreads();
  const int total = a.G << a.logM;
  const int shift = 32 - a.logM;
  for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
    int g = idx >> a.logM, j = idx & (a.M - 1);
    if (a.in_lines_fast) j = idx / a.G, g = idx - j * a.G;
    double2 v = make_double2(0.0, 0.0);
    if (first + g < a.lines && j < a.n) {
      v = fetch(a, off_in[g], j);
      if (BLUE) v = cmul(v, a.chirp[j]);
    }
    // the plain transform is decimation in time: it wants its input bit-reversed
    const int p = BLUE || a.logM == 0 ? j : (int)(__brev((unsigned)j) >> shift);
    lds[pad((g << a.logM) + p)] = v;
  }
  __syncthreads();
  if (BLUE) {
    all_stages<true>(lds, a, -1);
    for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
      const int p = idx & (a.M - 1);
      const int k = a.logM == 0 ? 0 : (int)(__brev((unsigned)p) >> shift);
      lds[pad(idx)] = cmul(lds[pad(idx)], a.bf[k]);
    }
    __syncthreads();
    all_stages<false>(lds, a, +1);
  } else {
    all_stages<false>(lds, a, a.sign);
  }
  const double inv_m = 1.0 / (double)a.M;
  const int stores = a.G * a.n_store;
  for (int idx = threadIdx.x; idx < stores; idx += blockDim.x) {
    // whole power-of-two lines (the common case) are decoded without a division
    int g = a.n_store == a.M ? idx >> a.logM : idx / a.n_store, k = idx - g * a.n_store;
    if (a.out_lines_fast) {
      k = idx / a.G, g = idx - k * a.G;
      if (first + g >= a.lines) continue;
    } else if (first + g >= a.lines) {
      break;
    }
    double2 v = lds[pad((g << a.logM) + k)];
    if (BLUE) {
      const double2 c = a.chirp[k];
      v = cmul(v, make_double2(c.x * inv_m, c.y * inv_m));
    }
    if (a.tw_total) {
      double sn, cs;
      sincospi(2.0 * (double)((int64_t)inner[g] * k) / (double)a.tw_total, &sn, &cs);
      v = cmul(v, make_double2(cs, a.sign > 0 ? sn : -sn));
    }
    store_elem(a.out.base, a.out.kind, off_out[g] + (int64_t)k * a.out.estride, v);
  }
}

// ── tables ──────────────────────────────────────────────────────────────────
__global__ void twiddle_kernel(double2 *tw, int M) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= M / 2) return;
  double sn, cs;
  sincospi(2.0 * (double)k / (double)M, &sn, &cs);  // k / M is exact or correctly rounded: M is a power of two
  tw[k] = make_double2(cs, -sn);
}

// exp(sign pi i j^2 / n) with j^2 reduced mod 2n in integers (nx_c_fft.c:656-663).
__global__ void chirp_kernel(double2 *c, int64_t n, int sign) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= n) return;
  const int64_t r = (j * j) % (2 * n);
  double sn, cs;
  sincospi((double)r / (double)n, &sn, &cs);
  c[j] = make_double2(cs, sign > 0 ? sn : -sn);
}

// The convolution filter conj(chirp[|d|]) wrapped to length M (nx_c_fft.c:665-710).
__global__ void chirp_filter_kernel(double2 *b, const double2 *chirp, int64_t n, int64_t M) {
  const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (d >= M) return;
  double2 v = make_double2(0.0, 0.0);
  if (d < n) v = chirp[d];
  else if (M - d < n) v = chirp[M - d];
  b[d] = make_double2(v.x, -v.y);
}

// ── workspace passes of the long transforms ─────────────────────────────────
struct StageArgs {
  Lines t;            // the tensor side
  double2 *w;         // workspace, [lines of this chunk][M]
  int64_t line0, lines;
  int64_t M, n, count;  // workspace line length; transform length; elements per line moved
  int n_load, load_mode, herm_s;
  const double2 *chirp;
  double scale;
};

__global__ __launch_bounds__(256) void stage_in_kernel(StageArgs s, FftArgs a) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= s.lines * s.M) return;
  const int64_t l = i / s.M, j = i - l * s.M;
  double2 v = make_double2(0.0, 0.0);
  if (j < s.n) {
    int unused;
    v = fetch(a, line_offset(s.t, s.line0 + l, &unused), (int)j);
    if (s.chirp) v = cmul(v, s.chirp[j]);
  }
  s.w[i] = v;
}

__global__ __launch_bounds__(256) void stage_out_kernel(StageArgs s) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= s.lines * s.count) return;
  const int64_t l = i / s.count, k = i - l * s.count;
  double2 v = s.w[l * s.M + k];
  if (s.chirp) {
    const double2 c = s.chirp[k];
    v = cmul(v, make_double2(c.x * s.scale, c.y * s.scale));
  }
  int unused;
  store_elem(s.t.base, s.t.kind, line_offset(s.t, s.line0 + l, &unused) + k * s.t.estride, v);
}

__global__ __launch_bounds__(256) void spectrum_mul_kernel(double2 *w, const double2 *bf, int64_t M, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  w[i] = cmul(w[i], bf[i % M]);
}

// ── host side ───────────────────────────────────────────────────────────────
static inline bool is_pow2(int64_t n) { return n > 0 && (n & (n - 1)) == 0; }
static inline int log2_of(int64_t n) {
  int l = 0;
  while ((int64_t(1) << l) < n) l++;
  return l;
}

enum TableKind : uint64_t { T_TWIDDLE = 1, T_CHIRP = 2, T_FILTER = 3 };
static inline uint64_t table_key(TableKind k, int64_t n, int sign) {
  return ((uint64_t)k << 60) | ((uint64_t)(sign > 0) << 59) | (uint64_t)n;
}

static int table_lookup(nxh_context *ctx, uint64_t key, size_t bytes, double2 **out, bool *fresh) {
  auto it = ctx->device_tables.find(key);
  if (it != ctx->device_tables.end()) {
    *out = (double2 *)it->second;
    *fresh = false;
    return NXH_OK;
  }
  // A table is filled by a kernel on the context's stream. While that stream is being
  // recorded the fill would only be recorded too: the table would count as present with
  // nothing in it, for every eager transform until the first replay, and every replay
  // would rewrite a table that other work reads. So a length is never first used there.
  if (ctx->capture)
    return nxh_fail(NXH_FAILURE, "fft",
                    "first use of this transform length while a graph is being captured: run it once eagerly first");
  void *p = nullptr;
  if (hipMalloc(&p, bytes ? bytes : 16) != hipSuccess) {
    (void)hipGetLastError();
    return nxh_fail(NXH_FAILURE, "fft", NXH_ERR_ALLOC);
  }
  ctx->device_tables[key] = p;
  *out = (double2 *)p;
  *fresh = true;
  return NXH_OK;
}

// Takes a table whose fill could not be queued out of the registry again.
static void table_drop(nxh_context *ctx, uint64_t key) {
  auto it = ctx->device_tables.find(key);
  if (it == ctx->device_tables.end()) return;
  (void)hipStreamSynchronize(ctx->stream);  // a fill kernel already queued may still write it
  (void)hipFree(it->second);
  ctx->device_tables.erase(it);
}

static int twiddles(nxh_context *ctx, int M, const double2 **out) {
  double2 *t;
  bool fresh;
  if (int rc = table_lookup(ctx, table_key(T_TWIDDLE, M, -1), (size_t)(M / 2) * sizeof(double2), &t, &fresh)) return rc;
  if (fresh && M >= 2) {
    hipLaunchKernelGGL(twiddle_kernel, dim3((M / 2 + 255) / 256), dim3(256), 0, ctx->stream, t, M);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) {
      table_drop(ctx, table_key(T_TWIDDLE, M, -1));
      return nxh_hip_fail("fft", e);
    }
  }
  *out = t;
  return NXH_OK;
}

static Lines workspace_lines(double2 *w, int64_t outer, int64_t outer_stride, int64_t innerdim, int64_t inner_stride,
                             int64_t estride) {
  Lines v{};
  v.base = (char *)w;
  v.kind = K_C64;
  v.nd = 2;
  v.dims[0] = outer;
  v.strides[0] = outer_stride;
  v.dims[1] = innerdim;
  v.strides[1] = inner_stride;
  v.estride = estride;
  return v;
}

static int launch_lines(nxh_context *ctx, FftArgs &a, bool blue) {
  // short lines share a workgroup of FFT_LDS_MIN elements; long ones get one each
  a.G = a.M >= FFT_LDS_MIN ? 1 : FFT_LDS_MIN / a.M;
  // strided lines whose neighbours are adjacent in memory: as many lines per workgroup as make
  // runs of 128 bytes, or as the LDS holds
  auto neighbours = [](const Lines &v) { return v.estride != 1 && v.nd >= 1 && v.strides[v.nd - 1] == 1 && v.dims[v.nd - 1] > 1; };
  a.in_lines_fast = neighbours(a.in);
  a.out_lines_fast = neighbours(a.out);
  if (a.in_lines_fast || a.out_lines_fast) a.G = std::max(1, std::min(FFT_LDS_MAX / a.M, std::max(16, FFT_LDS_MIN / a.M)));
  if ((int64_t)a.G > a.lines) a.G = (int)a.lines;
  if (a.G == 1) a.in_lines_fast = a.out_lines_fast = 0;
  const int64_t blocks = (a.lines + a.G - 1) / a.G;
  if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, "fft", "too many lines for one launch");
  const int64_t elems = (int64_t)a.G * a.M;
  const int threads = elems >= 8192 ? 1024 : elems >= 4096 ? 512 : 256;
  const size_t lds = (size_t)(elems + elems / 16 + 1) * sizeof(double2) + (size_t)a.G * (2 * sizeof(int64_t) + sizeof(int));
  auto kern = blue ? fft_lines_kernel<true> : fft_lines_kernel<false>;
  static std::once_flag once[2];
  static hipError_t attr_status[2] = {hipSuccess, hipSuccess};
  std::call_once(once[blue], [&] {
    attr_status[blue] = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)((FFT_LDS_MAX + FFT_LDS_MAX / 16) * sizeof(double2) + 4096));
  });
  NXH_HIP("fft", attr_status[blue]);
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(threads), lds, ctx->stream, a);
  NXH_HIP("fft", hipGetLastError());
  return NXH_OK;
}

// Power-of-two transform of `lines` contiguous complex128 lines of length M in
// the workspace `src`; the result lands in `dst` (src is overwritten).
static int pow2_workspace(nxh_context *ctx, double2 *src, double2 *dst, int64_t lines, int64_t M, int sign) {
  FftArgs a{};
  a.sign = sign;
  a.load_mode = LOAD_COMPLEX;
  if (M <= FFT_LDS_MAX) {
    a.in = workspace_lines(src, lines, M, 1, 0, 1);
    a.out = workspace_lines(dst, lines, M, 1, 0, 1);
    a.lines = lines;
    a.n = a.M = a.n_load = a.n_store = (int)M;
    a.logM = log2_of(M);
    if (int rc = twiddles(ctx, a.M, &a.tw)) return rc;
    return launch_lines(ctx, a, false);
  }
  const int lg = log2_of(M);
  const int64_t n1 = int64_t(1) << ((lg + 1) / 2), n2 = M / n1;
  if (n1 > FFT_LDS_MAX) return nxh_fail(NXH_FAILURE, "fft", "axis too long (the limit is 2^26 elements)");
  // x[j1 n2 + j2] -> X[k1 + n1 k2]: transforms of length n1 down the columns, a
  // twiddle exp(sign 2 pi i j2 k1 / M), transforms of length n2 along the rows
  a.in = a.out = workspace_lines(src, lines, M, n2, 1, n2);
  a.lines = lines * n2;
  a.n = a.M = a.n_load = a.n_store = (int)n1;
  a.logM = log2_of(n1);
  a.tw_total = M;
  if (int rc = twiddles(ctx, a.M, &a.tw)) return rc;
  if (int rc = launch_lines(ctx, a, false)) return rc;
  a.in = workspace_lines(src, lines, M, n1, n2, 1);
  a.out = workspace_lines(dst, lines, M, n1, 1, n1);
  a.lines = lines * n1;
  a.n = a.M = a.n_load = a.n_store = (int)n2;
  a.logM = log2_of(n2);
  a.tw_total = 0;
  if (int rc = twiddles(ctx, a.M, &a.tw)) return rc;
  return launch_lines(ctx, a, false);
}

struct Scratch {  // pool blocks released when the pass is done (stream-ordered reuse)
  nxh_context *ctx;
  void *p[2] = {nullptr, nullptr};
  ~Scratch() {
    for (void *q : p)
      if (q) nxh_free_locked(ctx, q);
  }
};

static int bluestein_tables(nxh_context *ctx, int64_t n, int64_t M, int sign, const double2 **chirp, const double2 **bf) {
  double2 *c, *f;
  bool fresh_c, fresh_f;
  if (int rc = table_lookup(ctx, table_key(T_CHIRP, n, sign), (size_t)n * sizeof(double2), &c, &fresh_c)) return rc;
  if (fresh_c) {
    hipLaunchKernelGGL(chirp_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, c, n, sign);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) {
      table_drop(ctx, table_key(T_CHIRP, n, sign));
      return nxh_hip_fail("fft", e);
    }
  }
  if (int rc = table_lookup(ctx, table_key(T_FILTER, n, sign), (size_t)M * sizeof(double2), &f, &fresh_f)) return rc;
  if (fresh_f) {
    // the filter counts as present only once every launch that fills it has been queued
    Scratch tmp{ctx};
    int rc = nxh_alloc_locked(ctx, (size_t)M * sizeof(double2), &tmp.p[0]);
    if (!rc) {
      hipLaunchKernelGGL(chirp_filter_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, ctx->stream,
                         (double2 *)tmp.p[0], c, n, M);
      if (hipError_t e = hipGetLastError(); e != hipSuccess) rc = nxh_hip_fail("fft", e);
    }
    if (!rc) rc = pow2_workspace(ctx, (double2 *)tmp.p[0], f, 1, M, -1);
    if (rc) {
      table_drop(ctx, table_key(T_FILTER, n, sign));
      return rc;
    }
  }
  *chirp = c;
  *bf = f;
  return NXH_OK;
}

// One axis pass: every line of `in` (n_load stored elements, read per
// `load_mode`) is transformed at length n and its first n_store bins are stored
// to `out` (their real parts when `out` is real). `in` and `out` may be the same tensor.
static int transform_lines(nxh_context *ctx, const Lines &in, const Lines &out, int64_t lines, int64_t n, int n_load,
                           int load_mode, int64_t n_store, int sign) {
  if (lines == 0 || n == 0 || n_store == 0) return NXH_OK;
  if (n > (int64_t(1) << 26)) return nxh_fail(NXH_FAILURE, "fft", "axis too long (the limit is 2^26 elements)");
  const bool blue = !is_pow2(n);
  const int64_t M = blue ? int64_t(1) << log2_of(2 * n - 1) : n;
  if (M > (int64_t(1) << 26)) return nxh_fail(NXH_FAILURE, "fft", "axis too long for a length that is not a power of two (the limit is 2^25 elements)");
  FftArgs a{};
  a.in = in;
  a.out = out;
  a.n = (int)n;
  a.n_load = n_load;
  a.load_mode = load_mode;
  a.herm_s = (int)n;
  a.n_store = (int)n_store;
  a.sign = sign;
  if (blue)
    if (int rc = bluestein_tables(ctx, n, M, sign, &a.chirp, &a.bf)) return rc;
  if (M <= FFT_LDS_MAX) {
    a.lines = lines;
    a.M = (int)M;
    a.logM = log2_of(M);
    if (int rc = twiddles(ctx, a.M, &a.tw)) return rc;
    return launch_lines(ctx, a, blue);
  }
  // long transform: chunks of lines through two workspaces
  const int64_t chunk = std::max<int64_t>(1, std::min(lines, FFT_WORK_ELEMS / M));
  Scratch ws{ctx};
  for (void *&p : ws.p)
    if (int rc = nxh_alloc_locked(ctx, (size_t)(chunk * M) * sizeof(double2), &p)) return rc;
  double2 *w0 = (double2 *)ws.p[0], *w1 = (double2 *)ws.p[1];
  for (int64_t l0 = 0; l0 < lines; l0 += chunk) {
    const int64_t nl = std::min(chunk, lines - l0);
    StageArgs s{};
    s.w = w0;
    s.line0 = l0;
    s.lines = nl;
    s.M = M;
    s.n = n;
    s.chirp = blue ? a.chirp : nullptr;
    s.t = in;
    const int64_t total = nl * M;
    if ((total + 255) / 256 > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, "fft", "too many elements for one launch");
    hipLaunchKernelGGL(stage_in_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, s, a);
    double2 *res = w1;
    if (int rc = pow2_workspace(ctx, w0, w1, nl, M, blue ? -1 : sign)) return rc;
    if (blue) {
      hipLaunchKernelGGL(spectrum_mul_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, w1, a.bf, M, total);
      if (int rc = pow2_workspace(ctx, w1, w0, nl, M, +1)) return rc;
      res = w0;
    }
    s.w = res;
    s.t = out;
    s.count = n_store;
    s.scale = 1.0 / (double)M;
    const int64_t stores = nl * n_store;
    hipLaunchKernelGGL(stage_out_kernel, dim3((unsigned)((stores + 255) / 256)), dim3(256), 0, ctx->stream, s);
    NXH_HIP("fft", hipGetLastError());
  }
  return NXH_OK;
}

static int complex_kind(int dtype) { return dtype == NXH_C32 ? K_C32 : dtype == NXH_C64 ? K_C64 : -1; }
static int real_kind(int dtype) { return dtype == NXH_F32 ? K_F32 : dtype == NXH_F64 ? K_F64 : -1; }

// The lines of `src` and `dst` along `axis` (axis < 0: every element is a line
// of length one), with the other dims merged where both tensors allow it.
static int make_lines(const char *op, const nxh_tensor *src, int src_kind, const nxh_tensor *dst, int dst_kind, int axis,
                      Lines *in, Lines *out, int64_t *lines) {
  *in = Lines{};
  *out = Lines{};
  in->base = (char *)src->data + src->offset * kind_size(src_kind);
  out->base = (char *)dst->data + dst->offset * kind_size(dst_kind);
  in->kind = src_kind;
  out->kind = dst_kind;
  in->estride = axis >= 0 ? src->strides[axis] : 0;
  out->estride = axis >= 0 ? dst->strides[axis] : 0;
  int nd = 0;
  *lines = 1;
  for (int d = 0; d < dst->ndim; d++) {
    if (d == axis || dst->shape[d] == 1) continue;
    const int64_t e = dst->shape[d];
    *lines *= e;
    if (nd > 0 && in->strides[nd - 1] == src->strides[d] * e && out->strides[nd - 1] == dst->strides[d] * e) {
      in->dims[nd - 1] *= e;
      out->dims[nd - 1] *= e;
      in->strides[nd - 1] = src->strides[d];
      out->strides[nd - 1] = dst->strides[d];
      continue;
    }
    if (nd == FFT_MAXD) return nxh_fail(NXH_FAILURE, op, "too many non-mergeable dims beside the transformed axis (the limit is 8)");
    in->dims[nd] = out->dims[nd] = e;
    in->strides[nd] = src->strides[d];
    out->strides[nd] = dst->strides[d];
    nd++;
  }
  in->nd = out->nd = nd;
  return NXH_OK;
}

static int check_axes(const char *op, const int32_t *axes, int n_axes, int ndim) {
  if (n_axes < 0 || (n_axes > 0 && !axes)) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  for (int i = 0; i < n_axes; i++)
    if (axes[i] < 0 || axes[i] >= ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXIS);
  return NXH_OK;
}

static int check_out(const char *op, const nxh_tensor *out) {
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  return NXH_OK;
}

static inline int length_as_int(const char *op, int64_t n) {
  return n > (int64_t(1) << 26) ? nxh_fail(NXH_FAILURE, op, "axis too long (the limit is 2^26 elements)") : NXH_OK;
}

}  // namespace

// nx_c_fft.c:940-956
NXH_EXPORT int nxh_fft(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const int32_t *axes, int n_axes,
                       int inverse) {
  NXH_DEFER_BARRIER(ctx, out);
  const char *op = inverse ? "ifft" : "fft";
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (!rc) rc = check_axes(op, axes, n_axes, x->ndim);
  if (!rc) rc = check_out(op, out);
  if (rc) return rc;
  const int kind = complex_kind(out->dtype);
  if (kind < 0 || x->dtype != out->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (!nxh_same_shape(out, x)) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path("fft_lines");
  const int passes = n_axes > 0 ? n_axes : 1;  // no axes: the transform over nothing, a copy
  for (int ai = 0; ai < passes; ai++) {
    const int axis = n_axes > 0 ? axes[ai] : -1;
    const nxh_tensor *src = ai == 0 ? x : out;
    const int64_t n = axis >= 0 ? out->shape[axis] : 1;
    if ((rc = length_as_int(op, n))) return rc;
    Lines in, o;
    int64_t lines;
    if ((rc = make_lines(op, src, kind, out, kind, axis, &in, &o, &lines))) return rc;
    if ((rc = transform_lines(ctx, in, o, lines, n, (int)n, LOAD_COMPLEX, n, inverse ? +1 : -1))) return rc;
  }
  return NXH_OK;
}

// nx_c_fft.c:958-982
NXH_EXPORT int nxh_rfft(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const int32_t *axes, int n_axes) {
  NXH_DEFER_BARRIER(ctx, out);
  const char *op = "rfft";
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (!rc) rc = check_axes(op, axes, n_axes, x->ndim);
  if (!rc) rc = check_out(op, out);
  if (rc) return rc;
  if (n_axes < 1) return nxh_fail(NXH_INVALID_ARGUMENT, op, "no axis to transform");
  const int ok = complex_kind(out->dtype), ik = real_kind(x->dtype);
  if (ok < 0 || ik < 0) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  const int last = axes[n_axes - 1];
  if (out->ndim != x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  const int64_t n = x->shape[last], half = n / 2 + 1;
  for (int d = 0; d < x->ndim; d++)
    if (out->shape[d] != (d == last ? half : x->shape[d])) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if ((rc = length_as_int(op, n))) return rc;
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path("fft_lines");
  Lines in, o;
  int64_t lines;
  if ((rc = make_lines(op, x, ik, out, ok, last, &in, &o, &lines))) return rc;
  if ((rc = transform_lines(ctx, in, o, lines, n, (int)n, LOAD_REAL, half, -1))) return rc;
  for (int ai = 0; ai < n_axes - 1; ai++) {
    const int axis = axes[ai];
    const int64_t m = out->shape[axis];
    if ((rc = length_as_int(op, m))) return rc;
    if ((rc = make_lines(op, out, ok, out, ok, axis, &in, &o, &lines))) return rc;
    if ((rc = transform_lines(ctx, in, o, lines, m, (int)m, LOAD_COMPLEX, m, -1))) return rc;
  }
  return NXH_OK;
}

// nx_c_fft.c:1029-1144
NXH_EXPORT int nxh_irfft(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const int32_t *axes, int n_axes,
                         int64_t s_last) {
  NXH_DEFER_BARRIER(ctx, out);
  const char *op = "irfft";
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (!rc) rc = check_axes(op, axes, n_axes, x->ndim);
  if (!rc) rc = check_out(op, out);
  if (rc) return rc;
  if (n_axes < 1) return nxh_fail(NXH_INVALID_ARGUMENT, op, "no axis to transform");
  const int ik = complex_kind(x->dtype), ok = real_kind(out->dtype);
  if (ok < 0 || ik < 0) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  const int last = axes[n_axes - 1];
  if (out->ndim != x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  const int64_t in_half = x->shape[last];
  const int64_t s = s_last > 0 ? s_last : 2 * (in_half - 1);
  for (int d = 0; d < x->ndim; d++)
    if (out->shape[d] != (d == last ? s : x->shape[d])) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if ((rc = length_as_int(op, s))) return rc;
  const int64_t half = std::min(in_half, s / 2 + 1);
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path("fft_lines");
  // the other axes first, in a contiguous complex128 temporary of x's shape
  nxh_tensor tmp = *x;
  Scratch hold{ctx};
  const nxh_tensor *src = x;
  int src_kind = ik;
  if (n_axes > 1) {
    int64_t count = 1;
    for (int d = x->ndim - 1; d >= 0; d--) {
      tmp.strides[d] = count;
      count *= x->shape[d];
    }
    if (count == 0 || s == 0) return NXH_OK;
    if ((rc = nxh_alloc_locked(ctx, (size_t)count * sizeof(double2), &hold.p[0]))) return rc;
    tmp.data = hold.p[0];
    tmp.offset = 0;
    tmp.dtype = NXH_C64;
    for (int ai = 0; ai < n_axes - 1; ai++) {
      const int axis = axes[ai];
      const int64_t m = x->shape[axis];
      if ((rc = length_as_int(op, m))) return rc;
      Lines in, o;
      int64_t lines;
      if ((rc = make_lines(op, src, src_kind, &tmp, K_C64, axis, &in, &o, &lines))) return rc;
      if ((rc = transform_lines(ctx, in, o, lines, m, (int)m, LOAD_COMPLEX, m, +1))) return rc;
      src = &tmp;
      src_kind = K_C64;
    }
  }
  Lines in, o;
  int64_t lines;
  // lines are counted over the output's other dims, which equal the input's
  if ((rc = make_lines(op, src, src_kind, out, ok, last, &in, &o, &lines))) return rc;
  return transform_lines(ctx, in, o, lines, s, (int)half, LOAD_HERMITIAN, s, +1);
}
