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
//   scan_cols   the case of scan_chunks that matters most, rows of a matrix with
//               unit-stride columns (cumsum along axis 0) in dtypes of at most four
//               bytes: one pass, the carries handed down between blocks (below).
// Float sums and products are reassociated by scan_rows (tolerance-level
// differences, inside the reference contract's 6x arithmetic tolerance for
// scans); integer results are exact.

#include "fold_common.hpp"
#include "stream_access.hpp"

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

// The same for few lines and many chunks (one long vector cut into thousands of chunks): a block
// per line, a lane per run of consecutive chunks; the lanes' totals meet in LDS. One lane per line
// walked the 4096 chunks of a 2^24-element vector one after the other: 0.3 of that scan's 0.44 ms.
template <class C, class CB>
__global__ __launch_bounds__(FOLD_THREADS) void scan_carry_block_kernel(C *carry, uint64_t n_lines, int chunks) {
  __shared__ C tot[FOLD_THREADS];
  const uint64_t line = blockIdx.x;
  const int per = (chunks + FOLD_THREADS - 1) / FOLD_THREADS;
  const int c0 = (int)threadIdx.x * per, c1 = c0 + per < chunks ? c0 + per : chunks;
  C s = CB::init();
  for (int c = c0; c < c1; c++) s = CB::apply(s, carry[(uint64_t)c * n_lines + line]);
  tot[threadIdx.x] = s;
  __syncthreads();
  C run = CB::init();
  for (int i = 0; i < (int)threadIdx.x; i++) run = CB::apply(run, tot[i]);
  for (int c = c0; c < c1; c++) {
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

// ── scan_narrow: a contiguous [rows][L] matrix with fewer than 16 columns, scanned down its rows ──
// (Running totals of a table of a few series.) Too narrow for scan_cols' strips of 256 columns,
// of which such a matrix fills a few lanes ([2^20, 10] f32: 942 us). The matrix is read as the flat
// run it is: the first (256 / L) * L lanes of a block take 256 / L whole rows per pass, lane t row
// t / L and column t % L of the pass, so neighbouring lanes touch neighbouring addresses. A pass's
// values meet in LDS, where a lane adds the rows above its own onto the column's running value.
// Blocks take runs of rows: PHASE 0 leaves each run's column totals, scan_narrow_carry_kernel
// turns them into what lies above each run, PHASE 2 scans the runs from there.
template <int DT, class CB, int PHASE>
__global__ __launch_bounds__(FOLD_THREADS) void scan_narrow_kernel(const void *in_v, void *out_v, int64_t R, int L,
                                                                  int64_t rows_per_block, void *carry_v) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  __shared__ C vals[FOLD_THREADS];
  __shared__ C run[16];
  const int per_pass = FOLD_THREADS / L, active = per_pass * L;
  const int t = threadIdx.x, col = t % L, row0 = t / L;
  const int64_t r_begin = (int64_t)blockIdx.x * rows_per_block;
  const int64_t rows = (r_begin + rows_per_block < R ? r_begin + rows_per_block : R) - r_begin;
  C *carry = (C *)carry_v + (int64_t)blockIdx.x * L;
  if (t < L) run[t] = PHASE == 2 ? carry[t] : CB::init();
  const S *in = (const S *)in_v + r_begin * L;
  S *out = (S *)out_v + r_begin * L;
  for (int64_t first = 0; first < rows; first += per_pass) {
    const bool live = t < active && first + row0 < rows;
    vals[t] = live ? TR::ld(in[first * L + t]) : CB::init();
    __syncthreads();
    C acc = CB::init();
    if (t < active) {
      acc = run[col];
      for (int j = 0; j <= row0; j++) acc = CB::apply(acc, vals[col + j * L]);
      if (PHASE == 2 && live) out[first * L + t] = TR::st(acc);
    }
    __syncthreads();
    // the last live row of the pass carries the column on
    const int64_t left = rows - first;
    const int last = (int)(left < per_pass ? left : per_pass) - 1;
    if (t < active && row0 == last) run[col] = acc;
  }
  if (PHASE == 0) {
    __syncthreads();
    if (t < L) carry[t] = run[t];
  }
}
// [blocks][L] run totals -> what lies above each run (an exclusive scan down the blocks), one lane
// per column, eight loads in flight.
template <class C, class CB>
__global__ __launch_bounds__(64) void scan_narrow_carry_kernel(C *carry, int blocks, int L) {
  const int c = threadIdx.x;
  if (c >= L) return;
  C above = CB::init();
  int b = 0;
  for (; b + 8 <= blocks; b += 8) {
    C t[8];
#pragma unroll
    for (int j = 0; j < 8; j++) t[j] = carry[(int64_t)(b + j) * L + c];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      carry[(int64_t)(b + j) * L + c] = above;
      above = CB::apply(above, t[j]);
    }
  }
  for (; b < blocks; b++) {
    const C t = carry[(int64_t)b * L + c];
    carry[(int64_t)b * L + c] = above;
    above = CB::apply(above, t);
  }
}

// ── scan_cols: the axis is the row dim of a [rows][columns] view with unit-stride columns ──
// One pass over the data. A block owns SC_ROWS rows of a strip of SC_COLS columns: every wave
// holds SC_RW rows x 4 columns per lane in registers, scans them down the rows, the waves'
// totals meet in LDS. What a block needs from the rows above it travels through `status`, one
// 64-bit (flag, value) word per column and row chunk, written and read with relaxed
// device-scope atomics (a word is complete by itself, so nothing has to be ordered around it):
// a block first publishes its own total (flag AGG), then walks the chunks above it from the
// nearest one up, adding totals until it meets one that already carries everything above it
// (flag PRE), and publishes that form of its own word; the words of up to SC_WIN chunks are
// requested together, so the way up costs one trip to memory per window, not per chunk. Block b
// is chunk b / nstrips of strip b % nstrips: the blocks a block waits for have smaller ids, were
// handed to the compute units before it, and publish their AGG word before they wait for
// anything. (An earlier form took its id from a ticket counter instead, which made that order
// a certainty, and paid for it with one more trip to memory in front of every block's first
// load: 55 against 49 us.) The wait is bounded all the same: past `spin_limit` polls that found
// nothing new a lane gives up on the words and adds the rows above it from the input itself.
// Flags carry the launch's epoch, so words of earlier launches read as "not there yet" and the
// block of words is never cleared between launches. Results that nothing reads back while
// they could still be cached are stored past the memory-side cache (the host's per-call
// decision, runtime.hip): the input then stays cached from one call to the next, which is worth
// more here than anything else ([4096,8192] f32: 63 -> 49 us; the three-pass form gains nothing
// from it).
constexpr int SC_RW = 16, SC_V = 4, SC_COLS = 64 * SC_V;
constexpr int SC_WIN = 16;  // chunks whose words a lane requests together on its way up
struct ScanColsArgs {
  const void *in;
  void *out;
  int64_t len, W, in_step, out_step;  // rows, columns, row pitches in elements
  uint32_t nstrips, epoch, spin_limit;
  uint32_t stream_out;  // the results go past the memory-side cache (decided per call on the host)
  uint64_t *status;     // [chunks][nstrips * SC_COLS]
};
// The 32 bits of a running value that travel in a word: a float as it is; an integer as its
// storage form (sums and products are modular and maxima stay inside the storage range, so the
// storage bits determine every later result).
template <class TR>
__device__ __forceinline__ uint32_t sc_pack(typename TR::C c) {
  using S = typename TR::S;
  if constexpr (std::is_same<typename TR::C, float>::value) {
    return __builtin_bit_cast(uint32_t, c);
  } else {
    return (uint32_t)(typename std::make_unsigned<S>::type)TR::st(c);
  }
}
template <class TR>
__device__ __forceinline__ typename TR::C sc_unpack(uint32_t u) {
  using S = typename TR::S;
  if constexpr (std::is_same<typename TR::C, float>::value) {
    return __builtin_bit_cast(float, u);
  } else {
    return TR::ld((S)(typename std::make_unsigned<S>::type)u);
  }
}
template <int DT>
constexpr bool scan_cols_ok() {
  using TR = Tr<DT>;
  return sizeof(typename TR::S) <= 4 &&
         ((TR::cat == CAT_FLOAT && std::is_same<typename TR::C, float>::value) || TR::cat == CAT_SINT || TR::cat == CAT_UINT);
}

// ORDERED (float sums and products, whose result depends on how the additions are nested): the
// way up takes a fixed shape instead of whatever is there first. Every SC_WIN-th chunk is an
// anchor; only anchors publish the PRE form; a lane takes the AGG words of the chunks down to
// the nearest anchor below it and that anchor's PRE word, for which it waits. The value a chunk
// starts from is then P(anchor) + (a + (b + ...)) over the chunks in between, the same nesting
// on every run. The other operations are exact and associative, any mix of words gives the
// same bits, and they keep taking what is there.
template <int DT, class CB, bool VEC, int SC_WAVES, bool ORDERED>
__global__ __launch_bounds__(64 * SC_WAVES) void scan_cols_kernel(ScanColsArgs a) {
  constexpr int SC_ROWS = SC_RW * SC_WAVES;
  static_assert(64 * SC_WAVES >= SC_COLS, "a lane per column in the hand-over");
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  // what a lane keeps per element between the two halves of the kernel: the running value
  // itself for floats, its storage form for integers (half the registers, same information)
  using K = typename std::conditional<std::is_same<C, float>::value, float, S>::type;
  __shared__ C tot[SC_WAVES][SC_COLS];
  __shared__ C pre[SC_COLS];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const uint32_t t = blockIdx.x;
  const uint32_t strip = t % a.nstrips, chunk = t / a.nstrips;
  const int c0 = lane * SC_V;
  const int64_t col = (int64_t)strip * SC_COLS + c0;
  const int64_t row0 = (int64_t)chunk * SC_ROWS + w * SC_RW;
  const int ncol = (int)(a.W - col >= SC_V ? SC_V : (a.W - col > 0 ? a.W - col : 0));
  const int nrow = (int)(a.len - row0 >= SC_RW ? SC_RW : (a.len - row0 > 0 ? a.len - row0 : 0));
  const S *p = (const S *)a.in + row0 * a.in_step + col;
  S *q = (S *)a.out + row0 * a.out_step + col;
  FVec<S, SC_V> x[SC_RW];
#pragma unroll
  for (int r = 0; r < SC_RW; r++) {
    if (r < nrow) {
      if (VEC && ncol == SC_V) {
        x[r] = *reinterpret_cast<const FVec<S, SC_V> *>(p + r * a.in_step);
      } else {
#pragma unroll
        for (int j = 0; j < SC_V; j++)
          if (j < ncol) x[r].v[j] = p[r * a.in_step + j];
      }
    }
  }
  K v[SC_RW][SC_V];
  C run[SC_V];
#pragma unroll
  for (int j = 0; j < SC_V; j++) run[j] = CB::init();
#pragma unroll
  for (int r = 0; r < SC_RW; r++)
#pragma unroll
    for (int j = 0; j < SC_V; j++) {
      if (r < nrow && j < ncol) run[j] = CB::apply(run[j], TR::ld(x[r].v[j]));
      if constexpr (std::is_same<C, float>::value) v[r][j] = run[j];
      else v[r][j] = TR::st(run[j]);
    }
#pragma unroll
  for (int j = 0; j < SC_V; j++) tot[w][c0 + j] = run[j];
  __syncthreads();
  if (threadIdx.x < SC_COLS) {
    // The block's first SC_COLS lanes take one column of the strip each through the hand-over.
    const int cme = threadIdx.x;
    C agg = tot[0][cme];
#pragma unroll
    for (int i = 1; i < SC_WAVES; i++) agg = CB::apply(agg, tot[i][cme]);
    C ex = CB::init();
    const uint64_t pitch = (uint64_t)a.nstrips * SC_COLS;
    uint64_t *mine = a.status + (uint64_t)chunk * pitch + (uint64_t)strip * SC_COLS + cme;
    const uint32_t f_agg = a.epoch * 2 + 1, f_pre = a.epoch * 2 + 2;
    if (chunk > 0) {
      __hip_atomic_store(mine, ((uint64_t)f_agg << 32) | sc_pack<TR>(agg), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // Walk up SC_WIN chunks at a time (their words are requested together: one trip to memory
      // per window, not per chunk) and take them nearest first while they are there.
      bool have = false, done = false, gave_up = false;
      uint32_t polls = 0;
      int64_t c = (int64_t)chunk - 1;
      while (c >= 0 && !done) {
        const int n = c + 1 < SC_WIN ? (int)(c + 1) : SC_WIN;
        uint64_t word[SC_WIN];
#pragma unroll
        for (int k = 0; k < SC_WIN; k++)
          if (k < n) word[k] = __hip_atomic_load(mine - (uint64_t)(chunk - c + k) * pitch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int took = 0;
#pragma unroll
        for (int k = 0; k < SC_WIN; k++) {
          if (k >= n || done || took != k) continue;
          const uint32_t f = (uint32_t)(word[k] >> 32);
          const bool anchor = ((c - k) % SC_WIN) == 0;
          if (ORDERED ? f != (anchor ? f_pre : f_agg) : (f != f_agg && f != f_pre)) continue;
          const C val = sc_unpack<TR>((uint32_t)word[k]);
          ex = have ? CB::apply(val, ex) : val;  // the earlier rows on the left
          have = true;
          done = ORDERED ? anchor : f == f_pre;
          took = k + 1;
        }
        c -= took;
        if (took == 0) {
          if (polls++ >= a.spin_limit) {
            gave_up = true;
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
      }
      if (gave_up) {  // the rows above, from the input itself
        const int64_t mycol = (int64_t)strip * SC_COLS + cme;
        ex = CB::init();
        if (mycol < a.W) {
          const S *top = (const S *)a.in + mycol;
          const int64_t above = (int64_t)chunk * SC_ROWS;
          for (int64_t r = 0; r < above; r++) ex = CB::apply(ex, TR::ld(top[r * a.in_step]));
        }
      }
    }
    const C incl = chunk > 0 ? CB::apply(ex, agg) : agg;
    if (!ORDERED || chunk % SC_WIN == 0)
      __hip_atomic_store(mine, ((uint64_t)f_pre << 32) | sc_pack<TR>(incl), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    pre[cme] = ex;
  }
  __syncthreads();
  // what lies above this wave's rows: the chunks above (pre) and the block's earlier waves
  C base[SC_V];
  const bool has_base = chunk > 0 || w > 0;
#pragma unroll
  for (int j = 0; j < SC_V; j++) {
    C b = CB::init();
    bool hb = false;
    if (chunk > 0) {
      b = pre[c0 + j];
      hb = true;
    }
    for (int i = 0; i < w; i++) {
      b = hb ? CB::apply(b, tot[i][c0 + j]) : tot[i][c0 + j];
      hb = true;
    }
    base[j] = b;
  }
#pragma unroll
  for (int r = 0; r < SC_RW; r++) {
    if (r < nrow) {
      FVec<S, SC_V> y;
#pragma unroll
      for (int j = 0; j < SC_V; j++) {
        C val;
        if constexpr (std::is_same<C, float>::value) val = v[r][j];
        else val = TR::ld(v[r][j]);
        y.v[j] = TR::st(has_base ? CB::apply(base[j], val) : val);
      }
      if (VEC && ncol == SC_V) {
        if (a.stream_out) store_stream(reinterpret_cast<FVec<S, SC_V> *>(q + r * a.out_step), y);
        else *reinterpret_cast<FVec<S, SC_V> *>(q + r * a.out_step) = y;
      } else {
#pragma unroll
        for (int j = 0; j < SC_V; j++)
          if (j < ncol) q[r * a.out_step + j] = y.v[j];
      }
    }
  }
}

// The device words of scan_cols, owned by the context: made (and cleared) on first use and when
// a launch needs more of them, cleared again only when the epoch counter runs out.
static int scan_cols_state(nxh_context *ctx, const char *op, size_t need) {
  if (need > ctx->scan_state_bytes) {
    if (ctx->scan_state) NXH_HIP(op, hipFree(ctx->scan_state));  // (waits for the device)
    ctx->scan_state = nullptr;
    ctx->scan_state_bytes = 0;
    const size_t bytes = std::max<size_t>(need, (size_t)8 << 20);
    void *p = nullptr;
    NXH_HIP(op, hipMalloc(&p, bytes));
    ctx->scan_state = (unsigned char *)p;
    ctx->scan_state_bytes = bytes;
    ctx->scan_epoch = 0x7fffffffu;  // forces the clearing below
  }
  if (ctx->scan_epoch >= 0x7ffffff0u) {
    NXH_HIP(op, hipMemsetAsync(ctx->scan_state, 0, ctx->scan_state_bytes, ctx->stream));
    ctx->scan_epoch = 0;
  }
  return NXH_OK;
}
static uint32_t scan_spin_limit() {
  static const uint32_t v = [] {
    const char *e = getenv("NXH_SCAN_SPIN");  // 0: every block takes the fallback (tests)
    return e ? (uint32_t)strtoul(e, nullptr, 10) : (uint32_t)(1u << 16);
  }();
  return v;
}

template <int OP, int DT>
static int scan_launch(nxh_context *ctx, const char *op, const nxh_tensor *in, const nxh_tensor *out,
                       const Geom &g, int64_t out_axis_stride, uint32_t stream) {
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
      if (g.n_out < 64 && chunks >= 64)
        hipLaunchKernelGGL((scan_carry_block_kernel<C, CB>), dim3((unsigned)g.n_out), dim3(FOLD_THREADS), 0, ctx->stream,
                           (C *)scratch.p[0], (uint64_t)g.n_out, (int)chunks);
      else
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
    // a contiguous matrix of fewer than 16 columns: read as one flat run (scan_narrow)
    if (g.nk == 1 && g.kin[0] == 1 && g.kout[0] == 1 && g.n_out >= 2 && g.n_out < 16 && a.in_step == g.n_out &&
        a.out_step == g.n_out && a.len >= 1024) {
      using C = typename TR::C;
      const int L = (int)g.n_out;
      const int64_t nblocks = std::min<int64_t>((int64_t)cus * 4, (a.len + 1023) / 1024);
      const int64_t rows_per_block = (a.len + nblocks - 1) / nblocks;
      const int64_t used = (a.len + rows_per_block - 1) / rows_per_block;
      Scratch scratch(ctx);
      int rc = scratch.get(0, (size_t)used * L * sizeof(C));
      if (rc) return rc;
      nxh_set_path("scan_narrow");
      const dim3 grid((unsigned)used), block(FOLD_THREADS);
      hipLaunchKernelGGL((scan_narrow_kernel<DT, CB, 0>), grid, block, 0, ctx->stream, (const void *)a.in, (void *)a.out, a.len, L,
                         rows_per_block, scratch.p[0]);
      hipLaunchKernelGGL((scan_narrow_carry_kernel<C, CB>), dim3(1), dim3(64), 0, ctx->stream, (C *)scratch.p[0], (int)used, L);
      hipLaunchKernelGGL((scan_narrow_kernel<DT, CB, 2>), grid, block, 0, ctx->stream, (const void *)a.in, (void *)a.out, a.len, L,
                         rows_per_block, scratch.p[0]);
      NXH_HIP(op, hipGetLastError());
      return NXH_OK;
    }
    if constexpr (scan_cols_ok<DT>()) {
      // columns with unit stride on both sides, too few of them for a lane each: one pass with
      // the carries handed down between blocks (not while a graph is captured: a replay would
      // meet its own epoch in the words)
      // 256, 128 or 64 rows per block: the tallest that still leaves two chunks. (Measured on
      // [4096,8192] f32: 16 waves 48.8 us, 8 waves 51.2; with 4 waves the chain of chunks is 64 long.)
      const int waves = a.len >= 512 ? 16 : a.len >= 256 ? 8 : 4;
      const int64_t rows_per_block = (int64_t)SC_RW * waves;
      const int64_t nstrips = (g.n_out + SC_COLS - 1) / SC_COLS, nchunks = (a.len + rows_per_block - 1) / rows_per_block;
      const size_t need = (size_t)nstrips * SC_COLS * (size_t)nchunks * sizeof(uint64_t);
      if (chunks >= 2 && g.nk == 1 && g.kin[0] == 1 && g.kout[0] == 1 && !ctx->capture && nchunks >= 2 &&
          in->data != out->data &&  // (a lane that gives up its wait reads input rows other blocks have long finished)
          nstrips * nchunks < ((int64_t)1 << 30) && need <= ((size_t)64 << 20)) {
        int rc = scan_cols_state(ctx, op, need);
        if (rc) return rc;
        ScanColsArgs c;
        c.in = a.in;
        c.out = a.out;
        c.len = a.len;
        c.W = g.n_out;
        c.in_step = a.in_step;
        c.out_step = a.out_step;
        c.nstrips = (uint32_t)nstrips;
        c.epoch = ++ctx->scan_epoch;
        c.spin_limit = scan_spin_limit();
        c.stream_out = (stream & NXH_STREAM_OUT) != 0;
        c.status = (uint64_t *)ctx->scan_state;
        const uint32_t nblocks = (uint32_t)(nstrips * nchunks);
        const uintptr_t al = (uintptr_t)(SC_V * sizeof(S)) - 1;
        const bool vec = !(((uintptr_t)a.in | (uintptr_t)a.out) & al) && a.in_step % SC_V == 0 && a.out_step % SC_V == 0;
        nxh_set_path("scan_cols");
        constexpr bool ORD = TR::cat == CAT_FLOAT && (OP == NXH_SUM || OP == NXH_PROD);
#define NXH_SCAN_COLS(WAVES)                                                                                         \
  do {                                                                                                               \
    if (vec) hipLaunchKernelGGL((scan_cols_kernel<DT, CB, true, WAVES, ORD>), dim3(nblocks), dim3(64 * WAVES), 0, ctx->stream, c); \
    else hipLaunchKernelGGL((scan_cols_kernel<DT, CB, false, WAVES, ORD>), dim3(nblocks), dim3(64 * WAVES), 0, ctx->stream, c);    \
  } while (0)
        if (waves == 4) NXH_SCAN_COLS(4);
        else if (waves == 8) NXH_SCAN_COLS(8);
        else NXH_SCAN_COLS(16);
#undef NXH_SCAN_COLS
        NXH_HIP(op, hipGetLastError());
        return NXH_OK;
      }
    }
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

typedef int (*scan_fn)(nxh_context *, const char *, const nxh_tensor *, const nxh_tensor *, const Geom &, int64_t, uint32_t);
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
  NXH_DEFER_SETTLE(ctx, 1, out, x);
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
  // whether the results go past the memory-side cache (only the single-pass column form asks)
  const void *base[2] = {out->data, x->data};
  uint64_t bytes[2] = {0, 0};
  for (int k = 0; k < 2; k++) {
    const nxh_tensor *t = k ? x : out;
    uint64_t n = 1;
    for (int d = 0; d < t->ndim; d++)
      if (t->strides[d] != 0) n *= (uint64_t)t->shape[d];
    bytes[k] = n * (uint64_t)nxh_elem_size(dt);
  }
  const uint32_t stream = nxh_cache_hints(ctx, 2, base, bytes, NXH_STREAM_OUT);
  return fn(ctx, name, x, out, g, out->strides[axis], stream);
}
